"""Router gating for MoE: softmax over the experts, top-k, optional renormalisation, on the library's kernel.

Call shape of the reference's builder (kernels/moe/topk_gating_softmax_kernel.py:392-686)::

    launch = build_topk_gating_softmax_module(num_experts=128, topk=6, dtype_str="bf16", renormalize=True)
    launch(gating, topk_weights, topk_indices, token_expert_indices, num_tokens, stream=stream)

``gating`` ``[tokens, num_experts]`` f32 / f16 / bf16; ``topk_weights`` fp32 and ``topk_indices`` / ``token_expert_indices``
4-byte elements (int32, or the fp32 views over int32 storage the reference's tests pass) ``[tokens, topk]``.  Ties go to
the lower expert index; ``token_expert_indices[t, k] = k * num_tokens + t``.  Any ``num_experts`` up to 1024 is accepted
(the reference needs ``num_experts / VPT`` to be a power of two, :42-62) and ``topk`` up to 32.
"""

from __future__ import annotations

import ctypes

import torch

from ... import _lib

_DTYPES = {"f32": (0, torch.float32), "bf16": (1, torch.bfloat16), "f16": (2, torch.float16)}


def gating_args(gating, weights, indices, tei, tokens, num_experts, topk, dtype_str, renormalize):
    """Checks the tensors and fills a ``psg_moe_gating_args``; ``weights`` / ``indices`` / ``tei`` may be ``None``."""
    if dtype_str not in _DTYPES:
        raise ValueError(f"dtype_str must be 'f32', 'f16' or 'bf16', got {dtype_str!r}")
    code, tdt = _DTYPES[dtype_str]
    if not gating.is_cuda or not gating.is_contiguous() or gating.dtype != tdt:
        raise ValueError(f"gating must be a contiguous {tdt} device tensor")
    if gating.numel() < tokens * num_experts:
        raise ValueError(f"gating holds {gating.numel()} elements, {tokens} tokens x {num_experts} experts need {tokens * num_experts}")
    a = _lib.MoeGatingArgs()
    a.gating = gating.data_ptr()
    for name, t in (("weights", weights), ("indices", indices), ("token_expert_indices", tei)):
        if t is None:
            continue
        if not t.is_cuda or not t.is_contiguous() or t.element_size() != 4 or t.device != gating.device:
            raise ValueError(f"{name} must be a contiguous device tensor of 4-byte elements on the device of gating")
        if name == "weights" and t.dtype != torch.float32:
            raise ValueError("weights must be float32")
        if t.numel() < tokens * topk:
            raise ValueError(f"{name} holds {t.numel()} elements, this call needs {tokens * topk}")
        setattr(a, name, t.data_ptr())
    a.tokens, a.experts, a.topk = int(tokens), int(num_experts), int(topk)
    a.dtype, a.renormalize = code, int(bool(renormalize))
    return a


class TopkGatingSoftmax:
    """Launcher returned by :func:`build_topk_gating_softmax_module`.  Holds no tensor references."""

    def __init__(self, num_experts, topk, dtype_str, renormalize):
        self.num_experts, self.topk, self.dtype_str, self.renormalize = int(num_experts), int(topk), dtype_str, bool(renormalize)
        self._lib = _lib.lib()

    def __call__(self, gating, topk_weights, topk_indices, token_expert_indices, num_tokens, stream=None):
        a = gating_args(gating, topk_weights, topk_indices, token_expert_indices, int(num_tokens), self.num_experts, self.topk,
                        self.dtype_str, self.renormalize)
        if not a.weights or not a.indices:
            raise ValueError("topk_weights and topk_indices must be given")
        rc = self._lib.psg_moe_topk_gating(ctypes.byref(a), _lib.stream_handle(stream))
        if rc:
            _lib.check(rc, "psg_moe_topk_gating")


def build_topk_gating_softmax_module(num_experts: int, topk: int, dtype_str: str = "bf16", renormalize: bool = True):
    """Same arguments as the reference's builder (:392-397); returns ``launch(gating, weights, indices, tei, num_tokens, *, stream)``."""
    if dtype_str not in _DTYPES:
        raise ValueError(f"dtype_str must be 'f32', 'f16' or 'bf16', got {dtype_str!r}")
    if not 1 <= int(num_experts) <= 1024:
        raise ValueError(f"num_experts={num_experts} is not supported: this kernel holds at most 1024 experts")
    if not 1 <= int(topk) <= min(32, int(num_experts)):
        raise ValueError(f"topk={topk} must lie in [1, min(32, num_experts)]")
    return TopkGatingSoftmax(num_experts, topk, dtype_str, renormalize)
