"""Routing of an expert layer (host side): which experts a token goes to, and with what weight.

Mirrors the two routing operators the reference registers for vLLM's ``_moe_C`` namespace next to
``moe_align_block_size`` and ``moe_sum``:
  topk_softmax   src/flag_gems/fused/topk_softmax.py:85-137 (kernel :24-82)
  grouped_topk   src/flag_gems/fused/grouped_topk.py:256-355 (kernels :25-78, :81-253)
with the same parameters, output tensors and errors.  Their results are the ``topk_weights`` / ``topk_ids`` that
``fused_experts_impl`` takes.
"""
from __future__ import annotations

import logging
from typing import Tuple

import torch

from . import _lib

logger = logging.getLogger("flag_gems." + __name__.split(".")[-1])

__all__ = ["topk_softmax", "grouped_topk"]

_SCORE_DTYPES = (torch.float32, torch.float16, torch.bfloat16)


def topk_softmax(
    topk_weights: torch.Tensor,
    topk_indices: torch.Tensor,
    token_expert_indices: torch.Tensor,
    gating_output: torch.Tensor,
    renormalize: bool = False,
) -> None:
    """Softmax over the experts and its ``topk`` largest probabilities per token, written into the caller's tensors:
    ``topk_weights [tokens, topk]`` fp32 (descending; divided by their sum with ``renormalize``), ``topk_indices`` (int32,
    uint32 or int64; ties go to the lower expert), ``token_expert_indices[t, k] = k * tokens + t`` (int32)."""
    logger.debug("GEMS TOPK SOFTMAX")
    num_tokens, num_experts = gating_output.shape
    topk = topk_weights.size(-1)
    assert topk <= 32
    if topk_indices.dtype not in (torch.int32, torch.uint32, torch.int64):
        raise TypeError("topk_indices must be int32/int64/uint32")
    if gating_output.dtype not in _SCORE_DTYPES:
        raise NotImplementedError(f"topk_softmax: unsupported gating dtype {gating_output.dtype}")
    if topk_weights.dtype != torch.float32 or token_expert_indices.dtype != torch.int32:
        raise NotImplementedError("topk_softmax: topk_weights must be float32 and token_expert_indices int32")
    for t in (topk_weights, topk_indices, token_expert_indices):
        assert t.shape == (num_tokens, topk) and t.is_contiguous()
    if num_tokens == 0 or topk == 0:
        return
    if gating_output.stride(1) != 1:
        gating_output = gating_output.contiguous()
    _lib.require_gpu(gating_output, "topk_softmax")
    with _lib.device_guard(gating_output.device):
        status = _lib.load().fg_topk_softmax(
            gating_output.data_ptr(), _lib.DTYPE_CODE[gating_output.dtype], num_tokens, num_experts,
            gating_output.stride(0) if num_tokens > 1 else max(num_experts, gating_output.stride(0)),
            topk, 1 if renormalize else 0, topk_weights.data_ptr(), topk_indices.data_ptr(), topk_indices.element_size(),
            token_expert_indices.data_ptr(), _lib.current_stream_ptr(gating_output.device))
    _lib.check(status, "fg_topk_softmax")


def grouped_topk(
    scores: torch.Tensor,
    n_group: int,
    topk_group: int,
    topk: int,
    renormalize: bool,
    routed_scaling_factor: float,
    bias: torch.Tensor,
    scoring_func: int = 0,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Group-limited routing: the ``topk`` experts with the largest ``score + bias`` among the ``topk_group`` groups
    whose two best biased scores sum highest; the weights are the scores (after the sigmoid when ``scoring_func`` is 1)
    times ``routed_scaling_factor``, divided by their sum with ``renormalize``.  Returns (fp32 ``[tokens, topk]``,
    int32 ``[tokens, topk]``)."""
    logger.debug("GEMS GROUPED TOPK")
    if scores.ndim != 2:
        raise ValueError("scores must be a 2D Tensor")
    num_tokens, num_experts = scores.shape
    if num_experts % n_group != 0:
        raise ValueError("num_experts must be divisible by n_group")
    if n_group > 32:
        raise ValueError("n_group should be smaller than or equal to 32")
    if topk > 32:
        raise ValueError("topk should be smaller than or equal to 32 for now")
    if scoring_func not in (0, 1):
        raise ValueError("scoring_func must be 0 (none) or 1 (sigmoid)")
    if bias.dtype != scores.dtype:
        bias = bias.to(scores.dtype)
    if bias.ndim != 1:
        bias = bias.flatten()
    if len(bias) != num_experts:
        raise ValueError(f"bias length ({len(bias)}) must match num_experts ({num_experts})")
    if scores.dtype not in _SCORE_DTYPES:
        raise ValueError(f"Unsupported dtype: {scores.dtype}")
    topk_values = torch.empty((num_tokens, topk), device=scores.device, dtype=torch.float32)
    topk_indices = torch.empty((num_tokens, topk), device=scores.device, dtype=torch.int32)
    if num_tokens == 0 or topk == 0:
        return topk_values, topk_indices
    if scores.stride(1) != 1:
        scores = scores.contiguous()
    bias = bias.contiguous()
    _lib.require_gpu(scores, "grouped_topk")
    with _lib.device_guard(scores.device):
        status = _lib.load().fg_grouped_topk(
            scores.data_ptr(), _lib.DTYPE_CODE[scores.dtype], num_tokens, num_experts,
            scores.stride(0) if num_tokens > 1 else max(num_experts, scores.stride(0)),
            bias.data_ptr(), n_group, topk_group, topk, 1 if renormalize else 0, float(routed_scaling_factor),
            int(scoring_func), topk_values.data_ptr(), topk_indices.data_ptr(), topk_values.stride(0),
            _lib.current_stream_ptr(scores.device))
    _lib.check(status, "fg_grouped_topk")
    return topk_values, topk_indices
