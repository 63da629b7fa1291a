"""Fused MX-FP4 MoE stages with the call shapes of the reference's ``kernels/moe/mxfp_moe`` (host.py:87-165
``flydsl_mxfp4_gemm1``, :168-231 ``flydsl_mxfp4_gemm2``).

Stage 1 multiplies the gathered token rows (MX-FP4, or MX-FP8 e4m3 with ``a_dtype="fp8"``) by the expert's gate and up rows
of W1 (MX-FP4), applies ``silu(gate) * up``, quantises the result to MX-FP4 again on the device and writes it by sorted
position; stage 2 multiplies those sorted rows by W2 and either adds ``weight * y`` atomically into the token's output row
(``epilog="atomic"``) or writes one unweighted row per sorted position (``epilog="nonatomic"`` / ``"nonatomic_cshuffle"``).

Built: ``BM`` 32 / 64 / 128 with pre-quantised activations, ``BM`` 16 with ``inline_quant=True`` (stage 1 reads the bf16
``hidden_states`` and quantises them itself; fp4 only) and, for stage 2, ``BM`` 16 as well; weights in the separate gate / up
row order (``interleave=False``).  ``use_nt``, ``BN``, ``BK`` and ``xcd_swizzle`` are tuning hints of the reference's kernels: they are
checked like the reference checks them and otherwise ignored.  Everything else raises ``NotImplementedError``, as the
reference does for the variants it does not build (host.py:142-146, :203-204).
"""

from __future__ import annotations

import ctypes

import torch

from ... import _lib

_A_DTYPE = {"fp4": 0, "fp8": 2}
_G2_EPILOGS = ("atomic", "nonatomic", "nonatomic_cshuffle")


def gemm1_grid(n_tokens, BM, *, NE, TOPK, INTER, BN=256):
    """Workgroups the reference launches for stage 1 (gemm1.py:59-67): blocks of ``BM`` sorted rows that can be in use, times
    the column blocks of the 2*INTER-wide output."""
    num_n_blocks = (2 * INTER + BN - 1) // BN
    if BM == 128:
        max_m_blocks = (n_tokens * TOPK + NE * (BM - 1) + BM - 1) // BM
    else:
        active = min(n_tokens * TOPK, NE)
        max_m_blocks = (n_tokens * TOPK + active * (BM - 1) + BM - 1) // BM
    return max_m_blocks * num_n_blocks


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _stream_handle(stream):
    if stream is None:
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if isinstance(stream, int):
        return ctypes.c_void_p(stream)
    return ctypes.c_void_p(stream.cuda_stream)


def _need(t, name, dtype=None, itemsize=None):
    """A pointer is all the library gets: refuse tensors whose element type, device or layout it would misread."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda or not t.is_contiguous():
        raise TypeError(f"{name} must be a contiguous device tensor")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if itemsize is not None and t.element_size() != itemsize:
        raise TypeError(f"{name} must have {itemsize}-byte elements, got {t.dtype}")


def _rows(t, row_bytes):
    return t.numel() * t.element_size() // row_bytes


def flydsl_mxfp4_gemm1(*, a_quant, a_scale_sorted_shuffled, w1_u8, w1_scale_u8, sorted_expert_ids, cumsum_tensor, m_indices,
                       inter_sorted_quant, inter_sorted_shuffled_scale, hidden_states=None, n_tokens, BM, use_nt=False,
                       inline_quant=False, NE, D_HIDDEN, D_INTER, topk, BN=256, BK=256, interleave=False, xcd_swizzle=0,
                       a_dtype="fp4", stream=None):
    """Stage 1.  ``m_indices`` holds the token of every sorted row (entries >= ``n_tokens`` are padding; the packed
    ``(slot << 24) | token`` ids of the sorter are accepted as they are).  Returns the two output tensors."""
    if D_HIDDEN % BK != 0:
        raise NotImplementedError(f"mxfp_moe gemm1 requires D_HIDDEN (K) % {BK} == 0, got H={D_HIDDEN}")
    if (2 * D_INTER) % BN != 0:
        raise NotImplementedError(f"mxfp_moe gemm1 requires 2*D_INTER (N_OUT) % {BN} == 0, got D_INTER={D_INTER}")
    inline_quant = bool(inline_quant)
    if interleave or a_dtype not in _A_DTYPE or (BM not in (32, 64, 128) if not inline_quant else (BM != 16 or a_dtype != "fp4")):
        raise NotImplementedError(
            f"mxfp_moe gemm1 unsupported variant (BM={BM}, use_nt={use_nt}, inline_quant={inline_quant}, interleave={interleave}, a_dtype={a_dtype})")
    if D_HIDDEN % 256 or D_INTER % 256:
        raise NotImplementedError(f"mxfp_moe gemm1 requires D_HIDDEN and D_INTER % 256 == 0, got {D_HIDDEN}, {D_INTER}")
    for t, name in ((m_indices, "m_indices"), (sorted_expert_ids, "sorted_expert_ids"), (cumsum_tensor, "cumsum_tensor")):
        _need(t, name, dtype=torch.int32)
    for t, name in ((w1_u8, "w1_u8"), (w1_scale_u8, "w1_scale_u8"), (inter_sorted_quant, "inter_sorted_quant"),
                    (inter_sorted_shuffled_scale, "inter_sorted_shuffled_scale")):
        _need(t, name, itemsize=1)
    if not inline_quant:
        _need(a_quant, "a_quant", itemsize=1)
        _need(a_scale_sorted_shuffled, "a_scale_sorted_shuffled", itemsize=1)
        a_row = int(D_HIDDEN) // 2 if a_dtype == "fp4" else int(D_HIDDEN)
        if _rows(a_quant, a_row) < int(n_tokens):
            raise ValueError(f"a_quant holds {_rows(a_quant, a_row)} rows of {a_row} bytes, n_tokens={n_tokens}")
        # the kernel's descriptor for these scales is sized from the sorted list, not from the tensor
        need_scale = (int(m_indices.numel()) + 31) // 32 * 32 * (int(D_HIDDEN) // 32)
        if a_scale_sorted_shuffled.numel() < need_scale:
            raise ValueError(f"a_scale_sorted_shuffled holds {a_scale_sorted_shuffled.numel()} bytes, the sorted list of "
                             f"{m_indices.numel()} rows needs ceil(rows / 32) * 32 * D_HIDDEN/32 = {need_scale}")
    if w1_u8.numel() < int(NE) * 2 * int(D_INTER) * (int(D_HIDDEN) // 2) or w1_scale_u8.numel() < int(NE) * 2 * int(D_INTER) * (int(D_HIDDEN) // 32):
        raise ValueError("w1_u8 / w1_scale_u8 are smaller than NE * 2*D_INTER rows of D_HIDDEN/2 code bytes and D_HIDDEN/32 scale bytes")
    sorted_size = int(m_indices.numel())
    args = _lib.MoeMxArgs()
    args.out, args.out_scale = _ptr(inter_sorted_quant), _ptr(inter_sorted_shuffled_scale)
    if inline_quant:
        if hidden_states is None or hidden_states.numel() < int(n_tokens) * int(D_HIDDEN):
            raise ValueError("inline_quant needs hidden_states: bf16 [n_tokens, D_HIDDEN]")
        _need(hidden_states, "hidden_states", dtype=torch.bfloat16)
        args.a, args.a_scale = _ptr(hidden_states), None
    else:
        args.a, args.a_scale = _ptr(a_quant), _ptr(a_scale_sorted_shuffled)
    args.w, args.w_scale = _ptr(w1_u8), _ptr(w1_scale_u8)
    args.sorted_token_ids, args.sorted_expert_ids = _ptr(m_indices), _ptr(sorted_expert_ids)
    args.sorted_weights, args.num_valid_ids = None, _ptr(cumsum_tensor)
    args.tokens, args.experts = int(n_tokens), int(NE)
    args.model_dim, args.inter_dim = int(D_HIDDEN), int(D_INTER)
    args.sorted_size = sorted_size
    args.blocks = min(int(sorted_expert_ids.numel()), sorted_size // int(BM))
    args.block_m, args.a_dtype, args.out_dtype = int(BM), 3 if inline_quant else _A_DTYPE[a_dtype], 0
    args.stage, args.atomic, args.pad0 = 1, 0, 0
    if _rows(inter_sorted_quant, D_INTER // 2) < sorted_size:
        raise ValueError(f"inter_sorted_quant holds {_rows(inter_sorted_quant, D_INTER // 2)} rows, the sorted list {sorted_size}")
    if inter_sorted_shuffled_scale.numel() < (sorted_size + 31) // 32 * 32 * (D_INTER // 32):
        raise ValueError("inter_sorted_shuffled_scale is smaller than ceil(sorted rows / 32) * 32 * D_INTER/32 bytes")
    lib = _lib.lib()
    _lib.check(lib.psg_moe_mx_gemm(ctypes.byref(args), _stream_handle(stream)), "psg_moe_mx_gemm (stage 1)")
    return inter_sorted_quant, inter_sorted_shuffled_scale


def flydsl_mxfp4_gemm2(*, inter_sorted_quant, inter_sorted_shuffled_scale, w2_u8, w2_scale_u8, sorted_expert_ids, cumsum_tensor,
                       sorted_token_ids, sorted_weights, flat_out, M_logical, max_sorted, BM, use_nt=False, epilog, NE, D_HIDDEN,
                       D_INTER, topk, flat_out_scale=None, D_INTER_REAL=None, BN=256, BK=256, xcd_swizzle=0, stream=None):
    """Stage 2.  ``flat_out`` is ``[M_logical, D_HIDDEN]`` (atomic; zeroed by the caller) or ``[max_sorted, D_HIDDEN]``
    (nonatomic), bf16 or fp16.  Returns ``flat_out``."""
    if D_INTER % BK != 0:
        raise NotImplementedError(f"mxfp_moe gemm2 contraction D_INTER (inter_dim) must be a multiple of {BK}, got D_INTER={D_INTER}")
    if D_HIDDEN % BN != 0:
        raise NotImplementedError(f"mxfp_moe gemm2 requires D_HIDDEN (N_OUT=model_dim) % {BN} == 0, got H={D_HIDDEN}")
    if epilog not in _G2_EPILOGS or BM not in (16, 32, 64, 128) or (D_INTER_REAL is not None and int(D_INTER_REAL) != int(D_INTER)):
        raise NotImplementedError(f"mxfp_moe gemm2 unsupported variant (BM={BM}, use_nt={use_nt}, epilog={epilog}, D_INTER_REAL={D_INTER_REAL})")
    if D_HIDDEN % 256 or D_INTER % 256:
        raise NotImplementedError(f"mxfp_moe gemm2 requires D_HIDDEN and D_INTER % 256 == 0, got {D_HIDDEN}, {D_INTER}")
    if flat_out.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"flat_out must be bf16 or fp16, got {flat_out.dtype}")
    for t, name in ((sorted_token_ids, "sorted_token_ids"), (sorted_expert_ids, "sorted_expert_ids"), (cumsum_tensor, "cumsum_tensor")):
        _need(t, name, dtype=torch.int32)
    _need(sorted_weights, "sorted_weights", dtype=torch.float32)
    for t, name in ((w2_u8, "w2_u8"), (w2_scale_u8, "w2_scale_u8"), (inter_sorted_quant, "inter_sorted_quant"),
                    (inter_sorted_shuffled_scale, "inter_sorted_shuffled_scale")):
        _need(t, name, itemsize=1)
    _need(flat_out, "flat_out")
    if w2_u8.numel() < int(NE) * int(D_HIDDEN) * (int(D_INTER) // 2) or w2_scale_u8.numel() < int(NE) * int(D_HIDDEN) * (int(D_INTER) // 32):
        raise ValueError("w2_u8 / w2_scale_u8 are smaller than NE * D_HIDDEN rows of D_INTER/2 code bytes and D_INTER/32 scale bytes")
    atomic = epilog == "atomic"
    max_sorted = int(max_sorted)
    need = (int(M_logical) if atomic else max_sorted) * int(D_HIDDEN)
    if flat_out.numel() < need:
        raise ValueError(f"flat_out holds {flat_out.numel()} elements, epilog {epilog!r} writes {need}")
    if sorted_token_ids.numel() < max_sorted or sorted_weights.numel() < max_sorted or _rows(inter_sorted_quant, D_INTER // 2) < max_sorted:
        raise ValueError("sorted_token_ids / sorted_weights / inter_sorted_quant are shorter than max_sorted rows")
    if inter_sorted_shuffled_scale.numel() < (max_sorted + 31) // 32 * 32 * (int(D_INTER) // 32):
        raise ValueError("inter_sorted_shuffled_scale is smaller than ceil(max_sorted / 32) * 32 * D_INTER/32 bytes")
    args = _lib.MoeMxArgs()
    args.out, args.out_scale = _ptr(flat_out), None
    args.a, args.a_scale = _ptr(inter_sorted_quant), _ptr(inter_sorted_shuffled_scale)
    args.w, args.w_scale = _ptr(w2_u8), _ptr(w2_scale_u8)
    args.sorted_token_ids, args.sorted_expert_ids = _ptr(sorted_token_ids), _ptr(sorted_expert_ids)
    args.sorted_weights, args.num_valid_ids = _ptr(sorted_weights), _ptr(cumsum_tensor)
    args.tokens, args.experts = int(M_logical), int(NE)
    args.model_dim, args.inter_dim = int(D_HIDDEN), int(D_INTER)
    args.sorted_size = max_sorted
    args.blocks = min(int(sorted_expert_ids.numel()), max_sorted // int(BM))
    args.block_m, args.a_dtype = int(BM), 0
    args.out_dtype = 0 if flat_out.dtype == torch.bfloat16 else 1
    args.stage, args.atomic, args.pad0 = 2, int(atomic), 0
    lib = _lib.lib()
    _lib.check(lib.psg_moe_mx_gemm(ctypes.byref(args), _stream_handle(stream)), "psg_moe_mx_gemm (stage 2)")
    return flat_out


def moe_mxfp4_sort(blockscale_e8m0, sorted_ids, num_valid_ids, token_num, block_size=32, out=None, stream=None):
    """The ``a_scale_sorted_shuffled`` input of stage 1 from the scales of the quantised activations, on the device in one launch
    (the reference's ``moe_mxfp4_sort``, tests/kernels/utils/gemm_common_utils.py:545-598, same arguments): ``blockscale_e8m0``
    ``[tokens, C]`` or ``[tokens, topk, C]`` bytes, ``C % 8 == 0``; returns ``[ceil(len(sorted_ids)/32)*32, C]`` uint8 (``out`` when
    given, which keeps the call allocation-free).  Rows of padding ids and rows past ``num_valid_ids[0]`` are zero."""
    if block_size % 32:
        raise AssertionError(f"block_size={block_size} must be a multiple of 32")
    _need(blockscale_e8m0, "blockscale_e8m0", itemsize=1)
    _need(sorted_ids, "sorted_ids", dtype=torch.int32)
    _need(num_valid_ids, "num_valid_ids", dtype=torch.int32)
    s = blockscale_e8m0.view(torch.uint8)
    if s.dim() not in (2, 3) or s.shape[0] < int(token_num) or s.shape[-1] % 8:
        raise ValueError(f"blockscale_e8m0 must be [tokens, C] or [tokens, topk, C] with C % 8 == 0 and at least token_num rows, got {tuple(s.shape)}")
    topk = 1 if s.dim() == 2 else int(s.shape[1])
    cols = int(s.shape[-1])
    if not s.is_contiguous():
        raise ValueError("blockscale_e8m0 must be contiguous")
    rows = (int(sorted_ids.numel()) + 31) // 32 * 32
    if out is None:
        out = torch.empty(rows, cols, dtype=torch.uint8, device=s.device)
    elif out.numel() * out.element_size() < rows * cols:
        raise ValueError(f"out holds {out.numel() * out.element_size()} bytes, {rows * cols} are written")
    lib = _lib.lib()
    _lib.check(lib.psg_moe_mx_scale_sort(_ptr(s), _ptr(sorted_ids), _ptr(num_valid_ids), _ptr(out), int(token_num), topk, cols, int(sorted_ids.numel()),
                                         _stream_handle(stream)), "psg_moe_mx_scale_sort")
    return out
