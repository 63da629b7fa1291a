"""Expert sorting of routed tokens, the layout the MoE stage kernels read.

Same outputs as the reference's torch-native sorter (tests/kernels/test_moe_gemm_2stage.py:99-137, itself a mirror of
aiter's ``moe_sorting``), computed without a Python loop over experts: one stable sort of the (token, slot) pairs by
expert, then a scatter into the padded positions.
"""

from __future__ import annotations

import torch


def moe_sorting(topk_ids: torch.Tensor, topk_weights: torch.Tensor, *, num_experts: int, block_size: int):
    """``topk_ids`` / ``topk_weights`` ``[tokens, topk]`` -> ``(sorted_ids int32, sorted_weights fp32, sorted_expert_ids
    int32, num_tokens_post_pad int32[2])``.

    ``sorted_ids[i] = (slot << 24) | token``; the rows of an expert are in (token, slot) order and padded to a multiple
    of ``block_size`` with ``(topk << 24) | tokens``; ``sorted_expert_ids`` holds one expert per block and -1 for the
    unused tail; ``num_tokens_post_pad = [padded rows in use, tokens]``.  Buffer sizes are the reference's upper bounds
    (``tokens*topk + experts*block_size - topk`` rows).  ``sorted_weights`` of padding rows is 0 here (the reference
    leaves it uninitialised).
    """
    if topk_ids.dim() != 2 or topk_ids.shape != topk_weights.shape:
        raise ValueError("topk_ids and topk_weights must both be [tokens, topk]")
    device = topk_ids.device
    tokens, topk = topk_ids.shape
    E, B = int(num_experts), int(block_size)
    if tokens >= 1 << 24:
        raise ValueError("token ids are packed into 24 bits")
    max_padded = int(tokens * topk + E * B - topk)
    max_blocks = (max_padded + B - 1) // B
    flat = topk_ids.reshape(-1).to(torch.int64)
    if flat.numel() and (int(flat.min()) < 0 or int(flat.max()) >= E):
        raise ValueError(f"expert ids must lie in [0, {E})")
    order = torch.sort(flat, stable=True).indices              # (token, slot) pairs grouped by expert, row-major inside
    counts = torch.bincount(flat, minlength=E)
    blocks_per = (counts + B - 1) // B
    start_padded = torch.cumsum(blocks_per * B, 0) - blocks_per * B
    start_dense = torch.cumsum(counts, 0) - counts
    exp_sorted = flat[order]
    pos = start_padded[exp_sorted] + (torch.arange(flat.numel(), device=device) - start_dense[exp_sorted])
    token = (order // topk).to(torch.int32)
    slot = (order % topk).to(torch.int32)
    sorted_ids = torch.full((max_padded,), (int(topk) << 24) | int(tokens), dtype=torch.int32, device=device)
    sorted_ids[pos] = (slot << 24) | token
    sorted_weights = torch.zeros((max_padded,), dtype=torch.float32, device=device)
    sorted_weights[pos] = topk_weights.reshape(-1).to(torch.float32)[order]
    sorted_expert_ids = torch.full((max_blocks,), -1, dtype=torch.int32, device=device)
    block_expert = torch.repeat_interleave(torch.arange(E, device=device, dtype=torch.int32), blocks_per)
    sorted_expert_ids[: block_expert.numel()] = block_expert
    num_tokens_post_pad = torch.stack([(blocks_per * B).sum(), torch.tensor(tokens, device=device)]).to(torch.int32)
    return sorted_ids, sorted_weights, sorted_expert_ids, num_tokens_post_pad
