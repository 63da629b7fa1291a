"""2-stage MoE GEMM entry points with the call shapes of the reference's ``kernels/moe/moe_gemm_2stage``:

    exe = compile_moe_gemm1(model_dim=..., inter_dim=..., experts=..., topk=..., tile_m=..., tile_n=..., tile_k=...,
                            doweight_stage1=False, out_dtype="f16", in_dtype="fp8")
    exe(out, x, w, scale_x, scale_w, sorted_token_ids, sorted_expert_ids, sorted_weights, num_valid_ids,
        tokens, inter_dim, model_dim, blocks, stream)

(gemm1.py:541-580 / launch_moe_gemm1 :502-537; gemm2.py:595-643; moe_reduce.py:164-203.)  ``x`` / ``w`` are fp8
(e4m3fn) or int8 with one fp32 scale per row; ``w`` is ``shuffle_weight`` of the experts' weights stacked along the
rows.  Built: ``in_dtype`` "fp8", "int8" and "int8smooth" (int8 whose stage-1 ``x`` / ``scale_x`` hold one row per (slot,
token), gemm1.py:100-101,321-328; stage 2 is plain int8) and "int4" (W4A8: int8 ``x``, ``w`` =
``flydsl_amd.layout.pack_shuffled_int8_to_int4(shuffle_weight(w_q))``, half the bytes; gemm1.py:41,170-189).  ``tile_m`` is the
block size of the expert sorting and must be 16, 32, 64 or 128; ``tile_n`` / ``tile_k`` are checked with the reference's
rules and then treated as hints.
"""

from __future__ import annotations

import ctypes

from ... import _lib

_OUT = {"f16": 1, "fp16": 1, "half": 1, "bf16": 0, "bfloat16": 0, "f32": 2, "fp32": 2, "float": 2}


def _check_tiles(stage, K, n_out, tile_m, tile_n, tile_k):
    # the reference's builder assertions (gemm1.py:56-72, gemm2.py:86-95)
    assert tile_k in (128, 256), f"stage {stage} needs tile_k in (128,256), got {tile_k}"
    if stage == 1:
        assert K % tile_k == 0 and (K // tile_k) % 2 == 0, f"K={K} must be an even multiple of TILE_K={tile_k}"
    else:
        assert K % tile_k == 0, f"K(inter_dim)={K} must be a multiple of TILE_K={tile_k}"
    assert 64 <= tile_n <= 256 and tile_n % 64 == 0, f"tile_n must be in [64,256] multiple of 64, got {tile_n}"
    assert 16 <= tile_m <= 256 and tile_m % 16 == 0, f"tile_m must be a 16-multiple in [16,256], got {tile_m}"
    contiguous_n = min(max(tile_n, 64), 128) if stage == 1 else tile_n
    assert n_out % contiguous_n == 0, f"output width {n_out} must be divisible by the channel tile {contiguous_n} (from tile_n={tile_n})"
    if tile_m not in (16, 32, 64, 128):
        raise ValueError(f"tile_m={tile_m}: this library sorts and multiplies in blocks of 16, 32, 64 or 128 rows")


class MoeStage:
    """Launcher of one stage.  Holds no tensor references."""

    def __init__(self, stage, model_dim, inter_dim, experts, topk, tile_m, doweight, out_dtype, accumulate, in_dtype):
        self.stage, self.model_dim, self.inter_dim = int(stage), int(model_dim), int(inter_dim)
        self.experts, self.topk, self.tile_m = int(experts), int(topk), int(tile_m)
        self.doweight, self.accumulate = bool(doweight), bool(accumulate)
        self.slot_major = in_dtype == "int8smooth" and int(stage) == 1
        self.w4 = in_dtype == "int4"
        self.no_pairing = False  # True: one workgroup per block of the sorted list even for blocks of 16 / 32 rows (tests)
        self.out_dtype, self.in_dtype = _OUT[str(out_dtype).strip().lower()], _lib.IN_DTYPE["int8" if in_dtype == "int8smooth" else in_dtype]
        self._lib = _lib.lib()

    def __call__(self, out, x, w, scale_x, scale_w, sorted_token_ids, sorted_expert_ids, sorted_weights, num_valid_ids,
                 tokens, dim0, dim1, blocks, stream=None):
        tokens, blocks = int(tokens), int(blocks)
        n_out, K = (self.inter_dim, self.model_dim) if self.stage == 1 else (self.model_dim, self.inter_dim)
        if (int(dim0), int(dim1)) != (n_out, K):
            raise ValueError(f"stage {self.stage} was built for dims ({n_out}, {K}), called with ({dim0}, {dim1})")
        rows_x = tokens if (self.stage == 1 and not self.slot_major) else tokens * self.topk
        rows_w = self.experts * (2 * n_out if self.stage == 1 else n_out)
        rows_out = tokens * self.topk if (self.stage == 1 or not self.accumulate) else tokens
        osize = 4 if self.out_dtype == 2 else 2
        dev = _lib.check_operand("out", out, min_elems=rows_out * n_out, elem_sizes=(osize,))
        _lib.check_operand("x", x, min_elems=rows_x * K, elem_sizes=(1,), device=dev)
        _lib.check_operand("w", w, min_elems=rows_w * K // (2 if self.w4 else 1), elem_sizes=(1,), device=dev)
        _lib.check_operand("scale_x", scale_x, min_elems=rows_x, elem_sizes=(4,), device=dev)
        _lib.check_operand("scale_w", scale_w, min_elems=rows_w, elem_sizes=(4,), device=dev)
        _lib.check_operand("sorted_token_ids", sorted_token_ids, min_elems=1, elem_sizes=(4,), device=dev)
        _lib.check_operand("sorted_expert_ids", sorted_expert_ids, min_elems=blocks, elem_sizes=(4,), device=dev)
        _lib.check_operand("sorted_weights", sorted_weights, min_elems=sorted_token_ids.numel() if self.doweight else 0, elem_sizes=(4,), device=dev)
        _lib.check_operand("num_valid_ids", num_valid_ids, min_elems=1, elem_sizes=(4,), device=dev)
        a = _lib.MoeArgs()
        a.out, a.x, a.w = out.data_ptr(), x.data_ptr(), w.data_ptr()
        a.scale_x, a.scale_w = scale_x.data_ptr(), scale_w.data_ptr()
        a.sorted_token_ids, a.sorted_expert_ids = sorted_token_ids.data_ptr(), sorted_expert_ids.data_ptr()
        a.sorted_weights, a.num_valid_ids = sorted_weights.data_ptr(), num_valid_ids.data_ptr()
        a.tokens, a.topk, a.experts = tokens, self.topk, self.experts
        a.model_dim, a.inter_dim = self.model_dim, self.inter_dim
        a.sorted_size, a.blocks, a.block_m = int(sorted_token_ids.numel()), blocks, self.tile_m
        a.in_dtype, a.out_dtype, a.stage = self.in_dtype, self.out_dtype, self.stage
        a.doweight, a.accumulate = int(self.doweight), int(self.accumulate)
        a.x_slot_major = int(self.slot_major)
        a.no_pairing = int(self.no_pairing)
        rc = self._lib.psg_moe_gemm(ctypes.byref(a), _lib.stream_handle(stream))
        if rc:
            _lib.check(rc, "psg_moe_gemm")


def _check_in_dtype(in_dtype):
    if in_dtype not in ("fp8", "int8", "int8smooth", "int4"):
        raise ValueError(f"in_dtype must be 'fp8', 'int8', 'int8smooth', or 'int4', got {in_dtype!r}")


def compile_moe_gemm1(*, model_dim: int, inter_dim: int, experts: int, topk: int, tile_m: int, tile_n: int, tile_k: int,
                      doweight_stage1: bool, out_dtype: str = "f16", in_dtype: str = "fp8"):
    """Stage 1 (gate-up + SiLU): kernels/moe/moe_gemm_2stage/gemm1.py:541-580, same keyword-only signature and errors."""
    if out_dtype not in ("f16", "bf16"):
        raise ValueError(f"out_dtype must be 'f16' or 'bf16', got {out_dtype!r}")
    _check_in_dtype(in_dtype)
    _check_tiles(1, int(model_dim), int(inter_dim), int(tile_m), int(tile_n), int(tile_k))
    return MoeStage(1, model_dim, inter_dim, experts, topk, tile_m, doweight_stage1, out_dtype, False, in_dtype)


def compile_moe_gemm2(*, model_dim: int, inter_dim: int, experts: int, topk: int, tile_m: int, tile_n: int, tile_k: int,
                      doweight_stage2: bool, out_dtype: str = "f16", accumulate: bool = True, in_dtype: str = "fp8"):
    """Stage 2 (down projection): kernels/moe/moe_gemm_2stage/gemm2.py:595-643, same keyword-only signature and errors."""
    out_s = str(out_dtype).strip().lower()
    if out_s not in _OUT:
        raise ValueError(f"out_dtype must be 'f16', 'bf16', or 'f32', got {out_dtype!r}")
    _check_in_dtype(in_dtype)
    if (not bool(accumulate)) and _OUT[out_s] == 2:
        raise ValueError("compile_moe_gemm2(accumulate=False) only supports out_dtype in {'f16','bf16'}")
    _check_tiles(2, int(inter_dim), int(model_dim), int(tile_m), int(tile_n), int(tile_k))
    return MoeStage(2, model_dim, inter_dim, experts, topk, tile_m, doweight_stage2, out_s, accumulate, in_dtype)


class MoeReduction:
    """Launcher returned by :func:`compile_moe_reduction`: ``(X, Y, expert_mask, topk_ids, m_tokens, stream)``."""

    def __init__(self, topk, model_dim, dtype, use_mask=False, num_experts=0):
        self.topk, self.model_dim, self.dtype = int(topk), int(model_dim), dtype
        self.use_mask, self.num_experts = bool(use_mask), int(num_experts)
        self._lib = _lib.lib()

    def __call__(self, X, Y, expert_mask, topk_ids, i32_m_tokens, stream=None):
        tokens = int(i32_m_tokens)
        esz = (4 if self.dtype == 2 else 2,)
        dev = _lib.check_operand("Y", Y, min_elems=tokens * self.model_dim, elem_sizes=esz)
        _lib.check_operand("X", X, min_elems=tokens * self.topk * self.model_dim, elem_sizes=esz, device=dev)
        if self.use_mask:
            # slots whose expert is masked out do not count (and their rows of X were never written)
            _lib.check_operand("expert_mask", expert_mask, min_elems=self.num_experts, elem_sizes=(4,), device=dev)
            _lib.check_operand("topk_ids", topk_ids, min_elems=tokens * self.topk, elem_sizes=(4,), device=dev)
            rc = self._lib.psg_moe_reduce_masked(X.data_ptr(), Y.data_ptr(), expert_mask.data_ptr(), topk_ids.data_ptr(), tokens, self.topk,
                                                 self.model_dim, self.num_experts, self.dtype, _lib.stream_handle(stream))
        else:
            rc = self._lib.psg_moe_reduce(X.data_ptr(), Y.data_ptr(), tokens, self.topk, self.model_dim, self.dtype, _lib.stream_handle(stream))
        if rc:
            _lib.check(rc, "psg_moe_reduce")


def compile_moe_reduction(*, topk: int, model_dim: int, dtype_str: str = "f16", use_mask: bool = False, num_experts: int = 0,
                          out_dtype_str: str | None = None):
    """Sum over the topk slots (kernels/moe/moe_gemm_2stage/moe_reduce.py:164-203), with ``use_mask`` only over the slots
    whose expert has ``expert_mask != 0`` (``num_experts`` entries).  Built for the dense variants f16 / bf16 / f32 (same
    input and output type, :57-61); the MXFP8 route-out rows (``dtype_str="fp8"``) raise ``NotImplementedError``."""
    if dtype_str not in ("f16", "bf16", "f32") or (out_dtype_str not in (None, dtype_str)):
        raise NotImplementedError("moe reduction is built for f16 / bf16 / f32, same type in and out")
    if use_mask and int(num_experts) < 1:
        raise ValueError("use_mask needs num_experts >= 1")
    return MoeReduction(topk, model_dim, _OUT[dtype_str], use_mask, num_experts)
