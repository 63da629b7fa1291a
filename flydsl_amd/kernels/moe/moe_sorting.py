"""Expert sorting of routed tokens, the layout the MoE stage kernels read.

Same outputs as the reference's sorters (kernels/moe/moe_sorting_kernel.py:2070-2215 ``moe_sorting_flydsl``; host
restatements tests/kernels/test_moe_sorting.py:74-110 and tests/kernels/test_moe_gemm_2stage.py:99-137).  Device
tensors go through the library's sorter kernel (``psg_moe_sorting``: one launch, no host synchronisation, records into
a graph); host tensors are sorted with torch (one stable sort of the (token, slot) pairs by expert, then a scatter).
"""

from __future__ import annotations

import ctypes

import torch

from ... import _lib

UNIT_SIZE = 32  # default rows per block, as in the reference (moe_sorting_kernel.py:43)


def sorted_sizes(tokens: int, topk: int, num_experts: int, block_size: int):
    """Upper bounds the reference sizes its buffers with: (rows of sorted_ids / sorted_weights, blocks)."""
    max_padded = int(tokens * topk + num_experts * block_size - topk)
    return max_padded, (max_padded + block_size - 1) // block_size


def moe_sorting_get_workspace_size(M, num_experts, topk, unit_size=UNIT_SIZE):
    """Bytes of workspace the sorter wants for ``M`` tokens (the reference's helper, moe_sorting_kernel.py:2030); 0 for
    routings small enough for the single launch."""
    return int(_lib.lib().psg_moe_sorting_workspace_bytes(int(M), int(topk), int(num_experts)))


def _sort_args(tokens, topk, sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf, num_experts, unit_size, expert_mask,
               workspace, device, routing=(), stream_h=0):
    """Checks the sorter's tensors and fills a ``psg_moe_sort_args`` (``routing`` = (topk_ids, topk_weights) when they are read).
    A workspace the caller did not bring comes from the library's pool for (device, stream ``stream_h``): those buffers are never
    released, so the up to three queued launches can still read it after this call has returned, whatever stream they run on
    (a tensor from the caching allocator would be handed to other work as soon as it is dropped here); the pool refuses to grow
    during graph capture."""
    E, B = int(num_experts), int(unit_size)
    need_rows, _ = sorted_sizes(tokens, topk, E, B)
    checks = [("sorted_ids", sorted_ids, torch.int32, need_rows), ("sorted_weights", sorted_weights, torch.float32, need_rows),
              ("sorted_expert_ids", sorted_expert_ids, torch.int32, (need_rows + B - 1) // B), ("num_valid_ids", num_valid_ids, torch.int32, 2)]
    if routing:
        checks += [("topk_ids", routing[0], torch.int32, tokens * topk), ("topk_weights", routing[1], torch.float32, tokens * topk)]
    if expert_mask is not None:
        checks.append(("expert_mask", expert_mask, torch.int32, E))
    for name, t, dt, n in checks:
        if not t.is_cuda or not t.is_contiguous() or t.dtype != dt:
            raise ValueError(f"{name} must be a contiguous {dt} device tensor")
        if t.numel() < n:
            raise ValueError(f"{name} holds {t.numel()} elements, this call needs at least {n}")
    if sorted_weights.numel() < sorted_ids.numel():
        raise ValueError("sorted_weights must be as long as sorted_ids")
    args = _lib.MoeSortArgs()
    if routing:
        args.topk_ids, args.topk_weights = routing[0].data_ptr(), routing[1].data_ptr()
    args.expert_mask = expert_mask.data_ptr() if expert_mask is not None else None
    args.sorted_ids, args.sorted_weights = sorted_ids.data_ptr(), sorted_weights.data_ptr()
    args.sorted_expert_ids, args.num_valid_ids = sorted_expert_ids.data_ptr(), num_valid_ids.data_ptr()
    if moe_buf is not None and moe_buf.numel():
        if not moe_buf.is_cuda or not moe_buf.is_contiguous():
            raise ValueError("moe_buf must be a contiguous device tensor")
        args.zero_buf, args.zero_bytes = moe_buf.data_ptr(), moe_buf.numel() * moe_buf.element_size()
    want = int(_lib.lib().psg_moe_sorting_workspace_bytes(tokens, topk, E))
    if workspace is None and want:
        workspace = _lib.workspace(device, want, stream_h, owner="moe_sort")
    if workspace is not None and workspace is not False:
        if not workspace.is_cuda or not workspace.is_contiguous():
            raise ValueError("workspace must be a contiguous device tensor")
        args.workspace, args.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    args.tokens, args.topk, args.experts, args.block_m = tokens, topk, E, B
    args.sorted_size = sorted_ids.numel()
    args.blocks = min(sorted_expert_ids.numel(), (sorted_ids.numel() + B - 1) // B)
    return args, workspace


def _local_tokens(num_local_tokens, rows):
    """The reference's ``num_local_tokens`` (moe_sorting_kernel.py:2100-2104): only the first so many rows are routed; a tensor is
    read with ``.item()`` (a host synchronisation, as in the reference), an int costs nothing."""
    if num_local_tokens is None:
        return int(rows)
    m = int(num_local_tokens.item()) if isinstance(num_local_tokens, torch.Tensor) else int(num_local_tokens)
    if not 1 <= m <= rows:
        raise ValueError(f"num_local_tokens={m} must lie in [1, {rows}]")
    return m


def moe_sorting_flydsl(topk_ids, topk_weights, sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf,
                       num_experts, unit_size=UNIT_SIZE, expert_mask=None, num_local_tokens=None, workspace=None, *,
                       stream=None):
    """The reference's call shape (moe_sorting_kernel.py:2070-2083): every output is pre-allocated by the caller and
    ``moe_buf`` (the buffer stage 2 accumulates into; may be ``None`` here) is cleared by the same launch.  ``topk_ids``
    int32 ``[tokens, topk]``, ``topk_weights`` fp32, ``expert_mask`` int32 ``[num_experts]`` or ``None``.  ``workspace``:
    a device tensor of ``moe_sorting_get_workspace_size(...)`` bytes lets routings of more than 4096 pairs sort in three
    short launches; ``None`` allocates one when it is needed (pass your own under graph capture or in serving loops),
    ``False`` forces the single launch.  ``num_local_tokens`` (int, or a tensor read with ``.item()``): sort only the first so
    many tokens; the padding value and ``num_valid_ids[1]`` then carry that count."""
    if topk_ids.dim() != 2 or topk_ids.shape != topk_weights.shape:
        raise ValueError("topk_ids and topk_weights must both be [tokens, topk]")
    tokens, topk = topk_ids.shape
    tokens = _local_tokens(num_local_tokens, tokens)
    stream_h = _lib.stream_handle(stream)
    args, _ws = _sort_args(tokens, topk, sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf, num_experts, unit_size,
                           expert_mask, workspace, topk_ids.device, routing=(topk_ids, topk_weights), stream_h=stream_h)
    handle = _lib.lib()
    rc = handle.psg_moe_sorting(ctypes.byref(args), stream_h)
    if rc != 0:
        raise (ValueError if rc < 0 else RuntimeError)(handle.psg_last_error().decode())
    return sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf


def moe_softmax_sort_flydsl(gating_logits, sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf, num_experts, topk,
                            dtype_str, unit_size=UNIT_SIZE, expert_mask=None, renormalize=True, num_local_tokens=None, *,
                            topk_ids=None, topk_weights=None, workspace=None, stream=None):
    """Router logits -> softmax -> top-k -> expert sort: the reference's fused entry point (moe_sorting_kernel.py:2250-2400),
    same positional arguments and the same outputs as ``moe_sorting_flydsl``.  For decode-sized batches (16 tokens with 256
    experts, 32 with up to 128) this is ONE launch (every sorting workgroup repeats the gating of all tokens in LDS; ``topk_ids`` / ``topk_weights`` are then optional extra
    outputs); beyond that the gating kernel and the sorter run back to back, through ``topk_ids`` / ``topk_weights`` when the
    caller gives them (``[tokens, topk]`` int32 / fp32) and through a buffer of the library's pool for this device and stream
    otherwise (never released, so the queued launches may outlive this call on any stream; the pool does not grow during
    graph capture: run the call once before capturing, or bring the tensors)."""
    from .topk_gating_softmax import gating_args

    if gating_logits.dim() != 2 or gating_logits.shape[1] != int(num_experts):
        raise ValueError("gating_logits must be [tokens, num_experts]")
    tokens, topk = _local_tokens(num_local_tokens, int(gating_logits.shape[0])), int(topk)
    handle = _lib.lib()
    fused = bool(handle.psg_moe_softmax_sorting_fused(tokens, topk, int(num_experts)))
    stream_h = _lib.stream_handle(stream)
    if not fused and (topk_ids is None or topk_weights is None):
        n = tokens * topk
        tmp = _lib.workspace(gating_logits.device, 8 * n, stream_h, owner="moe_softmax_sort")
        if topk_ids is None:
            topk_ids = tmp[: 4 * n].view(torch.int32).view(tokens, topk)
        if topk_weights is None:
            topk_weights = tmp[4 * n: 8 * n].view(torch.float32).view(tokens, topk)
    gargs = gating_args(gating_logits, topk_weights, topk_ids, None, tokens, int(num_experts), topk, dtype_str, renormalize)
    sargs, _ws = _sort_args(tokens, topk, sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf, num_experts, unit_size,
                            expert_mask, workspace, gating_logits.device, routing=() if fused else (topk_ids, topk_weights), stream_h=stream_h)
    rc = handle.psg_moe_softmax_sorting(ctypes.byref(gargs), ctypes.byref(sargs), stream_h)
    if rc != 0:
        raise (ValueError if rc < 0 else RuntimeError)(handle.psg_last_error().decode())
    return sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf


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
    max_padded, max_blocks = sorted_sizes(tokens, topk, E, B)
    if topk_ids.is_cuda:
        # the library's sorter kernel: no host synchronisation (expert ids outside [0, E) are dropped, not reported)
        out = (torch.empty(max_padded, dtype=torch.int32, device=device), torch.empty(max_padded, dtype=torch.float32, device=device),
               torch.empty(max_blocks, dtype=torch.int32, device=device), torch.empty(2, dtype=torch.int32, device=device))
        moe_sorting_flydsl(topk_ids.to(torch.int32).contiguous(), topk_weights.to(torch.float32).contiguous(), *out, None, E, B)
        return out
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
