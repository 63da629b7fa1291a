"""Host-side wire formats of the preshuffle GEMM (torch, any device).

The kernels read W as 1 KB blocks ``[N/16][Kbytes/64][klane 4][nlane 16][16 B]`` so that lane
``l = 16*klane + nlane`` of a wavefront fetches bytes ``[16 l, 16 l + 16)`` of a block as its MFMA
operand.  These helpers produce exactly the layouts of the reference's host utilities
(``shuffle_weight`` tests/utils.py:76-96; ``shuffle_weight_w4`` / ``shuffle_scale_w4``
tests/kernels/utils/gemm_common_utils.py:607-672) but are written from the closed-form byte map.
"""

from __future__ import annotations

import torch

_FP4X2 = getattr(torch, "float4_e2m1fn_x2", None)


def _blocked(x2d: torch.Tensor, rows_per_block: int, chunk_elems: int, chunks_per_block: int) -> torch.Tensor:
    """[R, C] -> blocks [R/rows][C/(chunk*chunks)][chunks][rows][chunk], flattened back to [R, C]."""
    r, c = x2d.shape
    cols_per_block = chunk_elems * chunks_per_block
    if r % rows_per_block or c % cols_per_block:
        raise AssertionError(f"shape {tuple(x2d.shape)} is not a multiple of ({rows_per_block}, {cols_per_block})")
    v = x2d.reshape(r // rows_per_block, rows_per_block, c // cols_per_block, chunks_per_block, chunk_elems)
    return v.permute(0, 2, 3, 1, 4).contiguous().reshape(r, c)


def shuffle_weight(x: torch.Tensor, layout=(16, 16), use_int4: bool = False) -> torch.Tensor:
    """Preshuffle ``W[..., N, K]``: element ``(n, k)`` moves to
    ``(n/16)*16K + (k/(2*IK*... ))`` -- for 1-byte elements byte offset
    ``(n/16)*16K + (k/32)*512 + ((k%32)/16)*256 + (n%16)*16 + k%16``; for 2-byte elements the chunk is
    8 elements.  Shape and dtype are kept; the result carries ``is_shuffled = True``."""
    x_type = x.dtype
    if _FP4X2 is not None and x_type == _FP4X2:
        x = x.view(torch.uint8)
    rows, ik = layout
    block_k = ik * 2
    chunk = 32 if use_int4 else 16 // x.element_size()
    n, k = x.shape[-2], x.shape[-1]
    assert n % rows == 0, f"{n} % {rows} == {n % rows}"
    assert k % block_k == 0, f"{k} % {block_k} == {k % block_k}"
    lead = x.shape[:-2]
    flat = x.reshape(-1, n, k)
    out = torch.stack([_blocked(m, rows, chunk, block_k // chunk) for m in flat]) if flat.shape[0] != 1 else _blocked(
        flat[0], rows, chunk, block_k // chunk
    ).unsqueeze(0)
    out = out.reshape(*lead, n, k).view(x_type)
    out.is_shuffled = True
    return out


def shuffle_weight_w4(src: torch.Tensor, NLane: int = 16, gate_up: bool = False, moe_gemm: bool = False) -> torch.Tensor:
    """Preshuffle packed fp4 bytes ``[N, K/2]`` into ``[N/16][Kpk/64][4][16][16 B]`` blocks."""
    if gate_up or moe_gemm:
        raise NotImplementedError("MoE / gate_up weight layouts are outside the preshuffle GEMM path")
    src_type = src.dtype
    if _FP4X2 is not None and src_type == _FP4X2:
        src = src.view(torch.uint8)
    klane = 64 // NLane
    return _blocked(src, NLane, 16, klane).view(src_type)


def shuffle_scale_w4(src: torch.Tensor, experts_cnt: int = 1, gate_up: bool = False) -> torch.Tensor:
    """Permute e8m0 scale bytes ``[R, K/32]`` so that byte ``(r, kb)`` lands at
    ``(r/32)*32*KB + (kb/8)*256 + (kb%4)*64 + (r%16)*4 + ((kb%8)/4)*2 + (r%32)/16``:
    one dword per lane per (32-row chunk, 256-K chunk), byte index = 2*(128-K half) + (16-row half)."""
    if gate_up or experts_cnt != 1:
        raise NotImplementedError("MoE scale layouts are outside the preshuffle GEMM path")
    r, kb = src.shape
    if r % 32 or kb % 8:
        raise AssertionError(f"scale shape {tuple(src.shape)} must be a multiple of (32, 8)")
    #            r/32   r half  r%16  kb/8   kb half  kb%4
    v = src.reshape(r // 32, 2, 16, kb // 8, 2, 4)
    #            r/32  kb/8  kb%4  r%16  kb half  r half
    return v.permute(0, 3, 5, 2, 4, 1).contiguous().reshape(r, kb)


def e8m0_shuffle(scale: torch.Tensor) -> torch.Tensor:
    """e8m0 scale bytes ``[R, C]`` padded to ``(ceil(R/256)*256, ceil(C/8)*8)`` and permuted like ``shuffle_scale_w4`` (the
    reference's ``e8m0_shuffle``, tests/kernels/utils/gemm_common_utils.py:114-136; the padding bytes are zero here, the
    reference leaves them uninitialised)."""
    if scale is None or scale.dtype == torch.float32:
        return scale
    assert scale.ndim == 2, "scale must be a 2D tensor"
    r, c = scale.shape
    pad = torch.zeros((r + 255) // 256 * 256, (c + 7) // 8 * 8, dtype=torch.uint8, device=scale.device)
    pad[:r, :c] = scale.view(torch.uint8)
    v = pad.view(pad.shape[0] // 32, 2, 16, pad.shape[1] // 8, 2, 4)
    return v.permute(0, 3, 5, 2, 4, 1).contiguous().view(pad.shape).view(scale.dtype)


def moe_mxfp4_sort(blockscale_e8m0: torch.Tensor, sorted_ids: torch.Tensor, num_valid_ids: torch.Tensor, token_num: int,
                   block_size: int = 32) -> torch.Tensor:
    """Scales of the SORTED rows of an MoE stage in the shuffled order its kernel reads (the reference's ``moe_mxfp4_sort``,
    tests/kernels/utils/gemm_common_utils.py:464-598): row ``i`` of the result's logical ``[rows, C]`` matrix is the scale
    row of token ``sorted_ids[i] & 0xFFFFFF`` (``[tokens, C]`` input) or of ``token * topk + (sorted_ids[i] >> 24)``
    (``[tokens, topk, C]`` input); padding rows and rows from ``num_valid_ids[0]`` on are zero (the reference leaves the
    latter unwritten).  Returns ``[ceil(rows/32)*32, C]`` bytes in the ``e8m0_shuffle`` order; ``C % 8 == 0``."""
    assert block_size % 32 == 0
    topk = 1
    s = blockscale_e8m0.view(torch.uint8)
    if s.dim() == 3:
        topk = s.shape[1]
        s = s.reshape(-1, s.shape[-1])
    rows_in, c = s.shape
    assert c % 8 == 0, f"{c} scale columns: a multiple of 8 is required"
    ids = sorted_ids.to(torch.int64)
    tok, slot = ids & 0xFFFFFF, (ids >> 24) & 0xFF
    src = tok if topk == 1 else tok * topk + slot
    live = (tok < token_num) & (torch.arange(ids.numel(), device=ids.device) < num_valid_ids.reshape(-1)[0].to(ids.device)) & (src < rows_in)
    rows = (ids.numel() + 31) // 32 * 32
    out = torch.zeros(rows, c, dtype=torch.uint8, device=s.device)
    out[: ids.numel()][live] = s[src[live]]
    v = out.view(rows // 32, 2, 16, c // 8, 2, 4)
    return v.permute(0, 3, 5, 2, 4, 1).contiguous().view(rows, c)


def pack_shuffled_int8_to_int4(x_shuf: torch.Tensor) -> torch.Tensor:
    """Packed int4 weights of the W4A8 MoE stages from PRESHUFFLED int8 values in [-8, 7]: every 8 consecutive values
    ``v0..v7`` become 4 bytes, ``byte j = (v_j & 15) | (v_{j+4} << 4)`` (low nibbles v0..v3, high nibbles v4..v7; the
    reference's ``_pack_shuffled_int8_to_packed_int4``, tests/kernels/test_moe_gemm_2stage.py:64-80).  Returns int8 of half
    the size, flat."""
    if x_shuf.dtype != torch.int8 or x_shuf.numel() % 8:
        raise ValueError("expected an int8 tensor whose size is a multiple of 8")
    v = x_shuf.contiguous().view(-1, 2, 4)
    if int(v.min()) < -8 or int(v.max()) > 7:
        raise ValueError("int4 weights must lie in [-8, 7]")
    lo = v[:, 0, :].to(torch.uint8) & 0xF
    hi = (v[:, 1, :].to(torch.uint8) & 0xF) << 4
    return (lo | hi).contiguous().view(-1).view(torch.int8)


def preshuffle_b(b_t: torch.Tensor) -> torch.Tensor:
    """Permute row-major 1-byte ``B_T [N, K]`` into the preshuffled fragment layout, as the reference's helper of the
    row-scale fp8 GEMMs does (kernels/gemm/fp8_gemm_utils.py:24-28): blocks ``[N/16][K/64][4][16][16 B]``, i.e. the
    byte map of ``shuffle_weight`` for 1-byte elements.  The result keeps that 5-D block shape."""
    n, k = b_t.shape[-2:]
    assert n % 16 == 0 and k % 64 == 0, f"need N%16==0 and K%64==0, got N={n} K={k}"
    return b_t.reshape(n // 16, 16, k // 64, 4, 16).permute(0, 2, 3, 1, 4).contiguous()
