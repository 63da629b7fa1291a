"""Shared helpers of the parity tests."""

from __future__ import annotations

import numpy as np
import torch

from flydsl_amd.synthetic import make_a8w8, make_a16w16, make_mx, make_mxfp4  # noqa: F401


def np_bytes(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.uint8).numpy()


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def np_u16(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)
