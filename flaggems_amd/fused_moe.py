"""A block-fp8 expert layer (host side): quantize -> grouped GEMM 1 -> SiLU-and-mul + quantize -> grouped GEMM 2
-> sum over the top-k slots.

Mirrors the block-wise fp8 configuration of the reference's ``fused_experts_impl``
(src/flag_gems/fused/fused_moe.py:1821-2185; ``use_fp8_w8a8=True`` with ``block_shape``), which its test states per
expert in torch (tests/test_fused_experts_impl.py:604-662).  The steps are the reference's:

  1. the activations are quantized per token and 128-group (``moe_kernel_quantize_input`` -> per_token_group_quant_fp8,
     fused_moe.py:674-683);
  2. GEMM 1 reads token ``slot // top_k`` for every routed slot (fused_moe.py:1111); the reference writes the result
     at the slot's own row (fused_moe.py:1484-1509), here it stays where it is computed, in expert order;
  3. SiLU-and-mul and the second quantization (fused_moe.py:2108-2122) -- one kernel here, row by row;
  4. GEMM 2 reads its rows (in place here, through the table in the reference), multiplies the fp32 sums by the slot's
     routing weight (``MUL_ROUTED_WEIGHT``, fused_moe.py:1495-1502) and writes every result at its slot's row;
  5. ``moe_sum`` adds the top-k slot rows of every token (fused_moe.py:2177-2182).

What differs is the routing table.  The reference pads every expert's rows to a multiple of the kernel's BLOCK_M
(``moe_align_block_size``); the grouped GEMM here takes arbitrary segment ends, so the slots are only sorted by
expert: ``moe_sort_slots`` returns the slot order and the cumulative ends, computed on the device without a
synchronisation.  Under expert parallelism (``expert_map``) the slots of experts that live elsewhere sort behind the
last segment, are never multiplied, and contribute zeros, as the reference's zero blocks do (fused_moe.py:1114).
"""
from __future__ import annotations

import logging
from typing import List, Optional, Tuple

import torch

from . import _lib
from .act_quant import per_token_group_quant_fp8, silu_and_mul_per_token_group_quant_fp8
from .grouped_block_fp8_matmul import grouped_w8a8_block_fp8_matmul

logger = logging.getLogger("flag_gems." + __name__.split(".")[-1])

_SORT_MAX_SLOTS = 65536   # limits of fg_moe_sort_slots
_SORT_MAX_EXPERTS = 960


def moe_sort_slots(
    topk_ids: torch.Tensor, num_experts: int, expert_map: Optional[torch.Tensor] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Routing table of an expert layer for ``grouped_w8a8_block_fp8_matmul``.

    ``topk_ids`` [T, top_k] holds an expert per routed slot; slot ``t * top_k + j`` is the j-th choice of token t.
    Returns ``(sorted_slots, offs)``: the slot numbers (int32 [T * top_k]) in ascending order of their local expert,
    ties in slot order, and the cumulative int32 ends of the ``num_experts`` local experts' segments.  With
    ``expert_map`` (global expert -> local expert or -1, the reference's convention:
    src/flag_gems/fused/moe_align_block_size.py:817-818) slots of experts that are not local sort last, behind
    ``offs[-1]``, as do slots whose id names no expert at all.  Everything stays on the device of ``topk_ids``; nothing
    synchronises.  Up to 65536 slots and 960 experts the table comes from one kernel (``fg_moe_sort_slots``, a stable
    counting sort in a single block); larger tables from torch's stable sort, with the same result.
    """
    flat = topk_ids.reshape(-1)
    n_slots = flat.numel()
    if (flat.is_cuda and n_slots <= _SORT_MAX_SLOTS and 1 <= num_experts <= _SORT_MAX_EXPERTS
            and flat.dtype in (torch.int32, torch.int64)
            and (expert_map is None or (expert_map.dtype in (torch.int32, torch.int64) and expert_map.device == flat.device))):
        # one kernel: a stable counting sort in a single block
        flat = flat.contiguous()
        emap = None if expert_map is None else expert_map.reshape(-1).contiguous()
        sorted_slots = torch.empty(n_slots, dtype=torch.int32, device=flat.device)
        offs = torch.empty(num_experts, dtype=torch.int32, device=flat.device)
        with _lib.device_guard(flat.device):
            status = _lib.load().fg_moe_sort_slots(
                flat.data_ptr(), flat.element_size(), n_slots, num_experts,
                None if emap is None else emap.data_ptr(), 0 if emap is None else emap.element_size(),
                0 if emap is None else emap.numel(), sorted_slots.data_ptr(), offs.data_ptr(),
                _lib.current_stream_ptr(flat.device))
        _lib.check(status, "fg_moe_sort_slots")
        return sorted_slots, offs
    # tables beyond the kernel's limits: the same table from torch's stable sort
    flat = flat.to(torch.int64)
    if expert_map is not None:
        inside = (flat >= 0) & (flat < expert_map.numel())
        flat = torch.where(inside, expert_map.reshape(-1).to(torch.int64)[flat.clamp(0, max(expert_map.numel() - 1, 0))],
                           torch.full_like(flat, -1))
    key = torch.where((flat >= 0) & (flat < num_experts), flat, torch.full_like(flat, num_experts))
    sorted_slots = torch.argsort(key, stable=True).to(torch.int32)
    counts = torch.zeros(num_experts + 1, dtype=torch.int64, device=flat.device)
    counts.scatter_add_(0, key, torch.ones_like(key))
    offs = torch.cumsum(counts[:num_experts], 0).to(torch.int32)
    return sorted_slots, offs


def moe_align_block_size_triton(
    topk_ids: torch.Tensor,
    num_experts: int,
    block_size: int,
    sorted_token_ids: torch.Tensor,
    expert_ids: torch.Tensor,
    num_tokens_post_pad: torch.Tensor,
) -> None:
    """The reference's in-place form under its own name (src/flag_gems/fused/moe_align_block_size.py:520-770; what
    vLLM's ``_moe_C::moe_align_block_size`` is patched with, src/flag_gems/patches/patch_vllm_all.py:306-321): fills
    the caller's three int32 buffers.  One kernel here, whatever the name says."""
    logger.debug("GEMS MOE ALIGN BLOCK SIZE")
    numel = topk_ids.numel()
    flat = topk_ids.reshape(-1)
    if not (flat.is_cuda and numel <= _SORT_MAX_SLOTS and 1 <= num_experts <= _SORT_MAX_EXPERTS
            and flat.dtype in (torch.int32, torch.int64)):
        raise NotImplementedError(
            f"moe_align_block_size: up to {_SORT_MAX_SLOTS} slots and {_SORT_MAX_EXPERTS} experts, int32 or int64 ids on the "
            f"GPU (got {numel} slots, {num_experts} experts, {flat.dtype} on {flat.device})")
    for t in (sorted_token_ids, expert_ids, num_tokens_post_pad):
        assert t.dtype == torch.int32 and t.is_contiguous() and t.device == flat.device
    assert num_tokens_post_pad.numel() >= 1
    flat = flat.contiguous()
    with _lib.device_guard(flat.device):
        status = _lib.load().fg_moe_align_block_size(
            flat.data_ptr(), flat.element_size(), numel, num_experts, block_size, sorted_token_ids.data_ptr(),
            sorted_token_ids.numel(), expert_ids.data_ptr(), expert_ids.numel(), num_tokens_post_pad.data_ptr(),
            _lib.current_stream_ptr(flat.device))
    _lib.check(status, "fg_moe_align_block_size")


def moe_align_block_size(
    topk_ids: torch.Tensor,
    block_size: int,
    num_experts: int,
    expert_map: Optional[torch.Tensor] = None,
    pad_sorted_ids: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """The reference's routing table (src/flag_gems/fused/moe_align_block_size.py:771-819): ``(sorted_ids, expert_ids,
    num_tokens_post_pad)`` with every expert's slots padded to a multiple of ``block_size`` by the value
    ``topk_ids.numel()``, the expert of every block (``expert_map`` applied, -1 where it has none) and the padded length.
    Same shapes as the reference allocates.  Inside an expert's run the slots are in ascending order (the reference's
    atomics leave that order open).  The expert layer of this package does not need this table (``moe_sort_slots``);
    it is here for callers that keep the reference's format, and ``local_rows_from_moe_align`` takes it from there."""
    numel = topk_ids.numel()
    cap = numel + num_experts * (block_size - 1)
    if pad_sorted_ids:
        cap = -(-cap // block_size) * block_size
    n_blocks = -(-cap // block_size)
    dev = topk_ids.device
    sorted_ids = torch.empty(cap, dtype=torch.int32, device=dev)
    expert_ids = torch.empty(n_blocks, dtype=torch.int32, device=dev)
    num_tokens_post_pad = torch.empty(1, dtype=torch.int32, device=dev)
    moe_align_block_size_triton(topk_ids, num_experts, block_size, sorted_ids, expert_ids, num_tokens_post_pad)
    if expert_map is not None:
        mapped = expert_map.reshape(-1).to(torch.int32)[expert_ids.clamp(min=0).long()]
        expert_ids = torch.where(expert_ids >= 0, mapped, expert_ids)
    return sorted_ids, expert_ids, num_tokens_post_pad


def moe_sum(input: torch.Tensor, output: torch.Tensor) -> None:
    """``output[t] = sum_k input[t, k]`` with an fp32 running sum in slot order and one rounding
    (src/flag_gems/fused/moe_sum.py:70-90)."""
    logger.debug("GEMS MOE SUM")
    assert input.ndim == 3 and output.ndim == 2
    tokens, top_k, hidden = input.shape
    assert output.shape == (tokens, hidden) and output.dtype == input.dtype and output.device == input.device
    if tokens == 0 or hidden == 0:
        return
    if input.stride(2) != 1:
        input = input.contiguous()
    assert output.stride(1) == 1
    _lib.require_gpu(input, "moe_sum")
    lib = _lib.load()
    with _lib.device_guard(input.device):
        status = lib.fg_moe_sum(
            input.data_ptr(), _lib.DTYPE_CODE[input.dtype], tokens, top_k, hidden, input.stride(0), input.stride(1),
            output.data_ptr(), output.stride(0), _lib.current_stream_ptr(input.device),
        )
    _lib.check(status, "fg_moe_sum")


def fused_experts_impl(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    inplace: bool = False,
    activation: str = "silu",
    apply_router_weight_on_input: bool = False,
    use_fp8_w8a8: bool = False,
    use_int8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    use_int4_w4a16: bool = False,
    ocp_mx_scheme: Optional[str] = None,
    per_channel_quant: bool = False,
    global_num_experts: int = -1,
    expert_map: Optional[torch.Tensor] = None,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    w1_zp: Optional[torch.Tensor] = None,
    w2_zp: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    block_shape: Optional[List[int]] = None,
    w1_bias: Optional[torch.Tensor] = None,
    w2_bias: Optional[torch.Tensor] = None,
    quant_scale_rule: str = "div",
) -> torch.Tensor:
    """The reference's signature (src/flag_gems/fused/fused_moe.py:1821-1847); served here: e4m3fn weights with
    128 x 128 block scales (``use_fp8_w8a8=True``, ``block_shape=[128, 128]``), SiLU, dynamic activation scales, no
    biases.  Every other configuration raises ``NotImplementedError``.

    hidden_states [T, H] bf16 / fp16; w1 [E, 2 I, H], w2 [E, H, I] e4m3fn; w1_scale [E, 2 I / 128, H / 128],
    w2_scale [E, H / 128, I / 128] fp32; topk_weights, topk_ids [T, top_k].  Returns [T, H] in the type of
    ``hidden_states`` (``inplace``: written into it).  ``quant_scale_rule`` (not in the reference's signature) picks
    the quantizer's scale formula: "div" is ``amax / 448`` with a true division of the elements, what the
    reference's kernel and the torch restatement in its MoE test compute (tests/test_fused_experts_impl.py:583-601).
    """
    logger.debug("GEMS FUSED MOE")
    assert activation == "silu", f"Only 'silu' activation is supported, got {activation}"
    if not use_fp8_w8a8 or use_int8_w8a8 or use_int8_w8a16 or use_int4_w4a16 or ocp_mx_scheme is not None:
        raise NotImplementedError("fused_experts_impl: only the block-wise fp8 configuration (use_fp8_w8a8=True) is built")
    if block_shape is None or list(block_shape) != [128, 128] or per_channel_quant:
        raise NotImplementedError("fused_experts_impl: fp8 weights need block_shape=[128, 128] (per-tensor and per-channel scales are not built)")
    if a1_scale is not None or a2_scale is not None:
        raise NotImplementedError("fused_experts_impl: static activation scales are not built")
    if w1_zp is not None or w2_zp is not None or w1_bias is not None or w2_bias is not None:
        raise NotImplementedError("fused_experts_impl: zero points and biases are not built")
    assert hidden_states.size(1) == w1.size(2), f"Hidden size mismatch {hidden_states.size(1)} != {w1.size(2)}"
    assert topk_weights.size() == topk_ids.size(), "topk shape mismatch"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.stride(-1) == 1, "Stride of last dimension must be 1"
    assert w2.stride(-1) == 1, "Stride of last dimension must be 1"
    assert hidden_states.dtype in [torch.float32, torch.float16, torch.bfloat16]
    assert w1_scale is not None and w2_scale is not None
    if hidden_states.dtype == torch.float32:
        raise NotImplementedError("fused_experts_impl: fp32 activations (the grouped GEMM writes bf16 or fp16)")

    T, H = hidden_states.shape
    E, N1, _ = w1.shape
    inter = N1 // 2
    assert w2.shape == (E, H, inter), f"w2 {tuple(w2.shape)} does not match w1 {tuple(w1.shape)}"
    top_k = topk_ids.size(1)
    out = hidden_states if inplace else torch.empty_like(hidden_states)
    if T == 0:
        return out
    dtype = hidden_states.dtype
    slots = T * top_k
    sorted_slots, offs = moe_sort_slots(topk_ids, E, expert_map)
    weights = topk_weights.reshape(-1).to(torch.float32).contiguous()

    xq, xs = per_token_group_quant_fp8(hidden_states, block_shape[1], scale_rule=quant_scale_rule)
    if apply_router_weight_on_input:
        # the routing weight multiplies GEMM 1's fp32 sums, which the kernel does where it scatters: both GEMMs read
        # and write slot rows, as the reference's kernel does
        cache1 = grouped_w8a8_block_fp8_matmul(
            xq, w1, xs, w1_scale, offs, block_shape, dtype, row_index=sorted_slots, index_divisor=top_k,
            scatter_rows=slots, row_weights=weights)
        aq, a_s = silu_and_mul_per_token_group_quant_fp8(cache1, block_shape[1], scale_rule=quant_scale_rule)
        cache3 = grouped_w8a8_block_fp8_matmul(
            aq, w2, a_s, w2_scale, offs, block_shape, dtype, row_index=sorted_slots, index_divisor=1,
            scatter_rows=slots, zero_unwritten_rows=expert_map is not None)
    else:
        # The rows between the two GEMMs stay in expert order: GEMM 1 gathers token sorted_slots[m] // top_k for sorted
        # row m and stores the row where it is (whole-line stores, no scatter), the activation and its quantizer work
        # row by row whatever the order, and GEMM 2 reads its rows in place and scatters sorted row m to slot row
        # sorted_slots[m], times the slot's routing weight.  Same values as with slot-ordered rows in between (the
        # reference's layout, fused_moe.py:1111, 1484-1509); rows of slots that no local expert serves are never
        # written by GEMM 1 (they lie behind the last segment), quantized like the rest and never read.
        cache1 = grouped_w8a8_block_fp8_matmul(
            xq, w1, xs, w1_scale, offs, block_shape, dtype, row_index=sorted_slots, index_divisor=top_k)
        aq, a_s = silu_and_mul_per_token_group_quant_fp8(cache1, block_shape[1], scale_rule=quant_scale_rule)
        cache3 = grouped_w8a8_block_fp8_matmul(
            aq, w2, a_s, w2_scale, offs, block_shape, dtype, row_index=sorted_slots, index_divisor=0,
            scatter_rows=slots, row_weights=weights, zero_unwritten_rows=expert_map is not None)
    moe_sum(cache3.view(T, top_k, H), out)
    return out


def inplace_fused_experts(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, topk_weights: torch.Tensor,
                          topk_ids: torch.Tensor, activation: str = "silu", **options) -> None:
    """``fused_experts_impl(..., inplace=True)``: the result replaces ``hidden_states``; returns nothing
    (src/flag_gems/fused/fused_moe.py:2188-2238; the remaining keywords are ``fused_experts_impl``'s)."""
    assert "inplace" not in options
    fused_experts_impl(hidden_states, w1, w2, topk_weights, topk_ids, inplace=True, activation=activation, **options)


def outplace_fused_experts(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, topk_weights: torch.Tensor,
                           topk_ids: torch.Tensor, activation: str = "silu", **options) -> torch.Tensor:
    """``fused_experts_impl(..., inplace=False)``: a new tensor (src/flag_gems/fused/fused_moe.py:2241-2291)."""
    assert "inplace" not in options
    return fused_experts_impl(hidden_states, w1, w2, topk_weights, topk_ids, inplace=False, activation=activation, **options)
