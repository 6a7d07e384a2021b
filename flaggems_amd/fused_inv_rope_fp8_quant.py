"""Inverse RoPE fused into the per-group FP8 quantizer (host side).

Mirrors ``fused_inv_rope_fp8_quant`` (src/flag_gems/fused/fused_inv_rope_fp8_quant.py:164-257): same parameters,
defaults, assertions and output layouts.  DeepSeek-V4 applies it to the attention output before the grouped output
projection, whose operands it lays out: ``o_fp8[:, g, :]`` is a contiguous ``[tokens, heads_per_group * head_dim]``
matrix for every group and the scales have unit stride along the tokens, which is what ``fp8_einsum("bhr,hdr->bhd")``
reads in place.
"""
from __future__ import annotations

import logging
from typing import Optional, Tuple

import torch

from . import _lib
from .act_quant import SUPPORTED_FP8_DTYPE, _IN_DTYPES

logger = logging.getLogger("flag_gems." + __name__.split(".")[-1])

__all__ = ["fused_inv_rope_fp8_quant"]


def _get_tma_aligned_size(size: int, align: int) -> int:
    return ((size + align - 1) // align) * align


def fused_inv_rope_fp8_quant(
    o: torch.Tensor,
    positions: torch.Tensor,
    cos_sin_cache: torch.Tensor,
    n_groups: int,
    heads_per_group: int,
    nope_dim: int = 448,
    rope_dim: int = 64,
    quant_group_size: int = 128,
    eps: float = 1e-10,
    dtype: Optional[torch.dtype] = None,
    tma_aligned_scales: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rotate the last ``rope_dim`` values of every head back by the token's position and quantize per group.

    o ``[num_tokens, num_heads, head_dim]``, positions ``[num_tokens]`` (int32 or int64), cos_sin_cache
    ``[max_position, rope_dim]`` fp32 laid out as cos || sin.  Returns ``o_fp8 [num_tokens, n_groups,
    heads_per_group * head_dim]`` with strides ``(d, num_tokens * d, 1)`` and ``o_scale [num_tokens, n_groups, blocks]``
    fp32 with unit stride along the tokens, or, with ``tma_aligned_scales``, int32 words of four UE8M0 exponents."""
    logger.debug("GEMS FUSED INV ROPE FP8 QUANT")

    fp8_dtype = SUPPORTED_FP8_DTYPE if dtype is None else dtype
    assert fp8_dtype == torch.float8_e4m3fn, "only torch.float8_e4m3fn is supported"
    assert o.ndim == 3, "`o` must be [num_tokens, num_heads, head_dim]"
    assert positions.ndim == 1, "`positions` must be 1D"
    assert cos_sin_cache.ndim == 2, "`cos_sin_cache` must be 2D"
    assert o.stride(-1) == 1, "head_dim must be contiguous"
    assert positions.shape[0] == o.shape[0], "positions and o token count mismatch"

    num_tokens, num_heads, head_dim = o.shape
    assert num_heads == n_groups * heads_per_group
    assert head_dim == nope_dim + rope_dim
    assert head_dim % quant_group_size == 0
    assert nope_dim % quant_group_size == (quant_group_size - rope_dim)
    assert rope_dim % 2 == 0
    assert cos_sin_cache.shape[-1] == rope_dim
    assert cos_sin_cache.dtype == torch.float32

    chunks_per_head = head_dim // quant_group_size
    if tma_aligned_scales:
        assert chunks_per_head <= 4, "packed UE8M0 path currently expects at most 4 scale blocks per head"

    d = heads_per_group * head_dim
    num_scale_blocks = d // quant_group_size
    tma_aligned_t = _get_tma_aligned_size(num_tokens, 4)
    if tma_aligned_scales:
        scale_inner, scale_dtype = (num_scale_blocks + 3) // 4, torch.int32
    else:
        scale_inner, scale_dtype = num_scale_blocks, torch.float32

    fp8_q = torch.empty((n_groups, num_tokens, d), dtype=fp8_dtype, device=o.device)
    scale = torch.empty(n_groups * scale_inner * tma_aligned_t, dtype=scale_dtype, device=o.device).as_strided(
        (n_groups, num_tokens, scale_inner), (scale_inner * tma_aligned_t, 1, tma_aligned_t))

    if o.dtype not in _IN_DTYPES:
        raise NotImplementedError(f"fused_inv_rope_fp8_quant: unsupported input dtype {o.dtype}")
    if positions.dtype not in (torch.int32, torch.int64):
        raise NotImplementedError(f"fused_inv_rope_fp8_quant: positions must be int32 or int64, got {positions.dtype}")
    if tma_aligned_scales and scale_inner != heads_per_group:
        # the reference's packed store writes one word per head at column head_in_group: with fewer than four groups per
        # head its columns would not line up with the (blocks + 3) // 4 it allocates
        raise NotImplementedError("fused_inv_rope_fp8_quant: packed scales need four groups per head")
    if num_tokens > 0 and num_heads > 0:
        _lib.require_gpu(o, "fused_inv_rope_fp8_quant")
        positions = positions.contiguous()
        if cos_sin_cache.stride(1) != 1:
            cos_sin_cache = cos_sin_cache.contiguous()
        with _lib.device_guard(o.device):
            status = _lib.load().fg_inv_rope_group_quant_fp8(
                o.data_ptr(), _lib.DTYPE_CODE[o.dtype], num_tokens, num_heads, head_dim, o.stride(0), o.stride(1),
                positions.data_ptr(), positions.element_size(),
                cos_sin_cache.data_ptr(), cos_sin_cache.shape[0], cos_sin_cache.stride(0),
                heads_per_group, rope_dim, quant_group_size, float(eps),
                fp8_q.data_ptr(), fp8_q.stride(0), fp8_q.stride(1),
                scale.data_ptr(), scale.stride(0), scale.stride(2),
                tma_aligned_t, 1 if tma_aligned_scales else 0, _lib.current_stream_ptr(o.device))
        _lib.check(status, "fg_inv_rope_group_quant_fp8")

    return fp8_q.transpose(0, 1), scale.transpose(0, 1)
