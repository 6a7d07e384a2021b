"""RMSNorm, with or without the residual add, alone or fused into the per-token-group FP8 quantizer.

The reference normalises with ``rms_norm`` (src/flag_gems/ops/rms_norm.py:54-66) or ``fused_add_rms_norm``
(src/flag_gems/fused/fused_add_rms_norm.py:92-145) and quantizes afterwards inside the fp8 linear layer
(src/flag_gems/ops/per_token_group_quant_fp8.py:203-297).  Here one HIP kernel does both, and the same kernel with
the quantizer switched off serves the two norm operators, so the fused result equals the two-step result bit for bit.
"""
from __future__ import annotations

import logging
import math
from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from .act_quant import (
    SUPPORTED_FP8_DTYPE,
    _FP8_DTYPES,
    _IN_DTYPES,
    _default_rule_and_floor,
    _round_to_dtype,
    _scale_rule_code,
)

logger = logging.getLogger(__name__)

__all__ = ["rms_norm", "rms_norm_out", "fused_add_rms_norm", "rms_norm_per_token_group_quant_fp8"]


def _launch(x2d, residual2d, weight, eps, y2d, q2d, s2d, group_size, quant_eps, fp8_dtype, scale_rule, scale_ue8m0):
    rows, cols = x2d.shape
    if weight.dtype != x2d.dtype or weight.numel() != cols or not weight.is_contiguous():
        raise NotImplementedError("RMSNorm: weight must be a contiguous vector of the input's dtype and row length")
    if x2d.dtype not in _IN_DTYPES:
        raise NotImplementedError(f"RMSNorm: unsupported input dtype {x2d.dtype}")
    _lib.require_gpu(x2d, "RMSNorm")

    def stride(t):
        return t.stride(0) if rows > 1 else max(cols, t.stride(0))

    if q2d is not None:
        finfo = torch.finfo(fp8_dtype)
        if scale_rule is None:  # the process-wide default of per_token_group_quant_fp8, whose twin the fused call is
            rule_code, floor = _default_rule_and_floor(quant_eps, x2d.dtype)
        else:
            rule_code, floor = _scale_rule_code(scale_rule), _round_to_dtype(float(quant_eps), x2d.dtype)
        qargs = (q2d.data_ptr(), _lib.DTYPE_CODE[fp8_dtype], stride(q2d), s2d.data_ptr(), s2d.stride(0), s2d.stride(1),
                 group_size, floor, finfo.min, finfo.max, 1.0 / finfo.max,
                 rule_code, _lib.FG_QUOT_DIV, _lib.FG_POW2_LOG2 if scale_ue8m0 else _lib.FG_POW2_NONE)
    else:
        qargs = (None, 0, 0, None, 0, 0, 0, 0.0, 0.0, 0.0, 0.0, 0, 0, 0)
    with _lib.device_guard(x2d.device):
        status = _lib.load().fg_rms_norm_group_quant_fp8(
            x2d.data_ptr(), _lib.DTYPE_CODE[x2d.dtype], rows, cols, stride(x2d),
            residual2d.data_ptr() if residual2d is not None else None, stride(residual2d) if residual2d is not None else 0,
            weight.data_ptr(), float(eps),
            y2d.data_ptr() if y2d is not None else None, stride(y2d) if y2d is not None else 0,
            *qargs, _lib.current_stream_ptr(x2d.device))
    _lib.check(status, "fg_rms_norm_group_quant_fp8")


def _rows_of(x: torch.Tensor, normalized_shape: Sequence[int]) -> Tuple[int, int]:
    dim = x.ndim - len(normalized_shape)
    assert tuple(x.shape[dim:]) == tuple(normalized_shape), "normalized_shape must be the trailing dimensions of x"
    return math.prod(x.shape[:dim]), math.prod(normalized_shape)


def rms_norm(x: torch.Tensor, normalized_shape: Sequence[int], weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """``weight * x / sqrt(mean(x^2) + eps)`` over the trailing ``normalized_shape``
    (src/flag_gems/ops/rms_norm.py:54-66: the normalised value is rounded to x's dtype before the weight)."""
    logger.debug("GEMS RMS_NORM FORWARD")
    rows, cols = _rows_of(x, normalized_shape)
    x = x.contiguous()
    y = torch.empty_like(x)
    if x.numel():
        _launch(x.view(rows, cols), None, weight.contiguous(), eps, y.view(rows, cols), None, None, 0, 0.0, None, None, False)
    return y


def rms_norm_out(result: torch.Tensor, x: torch.Tensor, normalized_shape: Sequence[int], weight: torch.Tensor,
                 eps: float = 1e-5) -> torch.Tensor:
    """``rms_norm`` into ``result`` (x's shape and dtype, contiguous): what vLLM's ``_C::rms_norm(result, input, weight,
    epsilon)`` asks for (src/flag_gems/patches/patch_vllm_all.py:610-613)."""
    logger.debug("GEMS RMS_NORM OUT")
    rows, cols = _rows_of(x, normalized_shape)
    assert result.shape == x.shape and result.dtype == x.dtype and result.device == x.device and result.is_contiguous()
    x = x.contiguous()
    if x.numel():
        _launch(x.view(rows, cols), None, weight.contiguous(), eps, result.view(rows, cols), None, None, 0, 0.0, None, None, False)
    return result


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, normalized_shape: Sequence[int], weight: torch.Tensor,
                       eps: float = 1e-5) -> Tuple[torch.Tensor, torch.Tensor]:
    """In place: ``residual += x`` (summed in fp32), ``x = rms_norm(that sum) * weight``
    (src/flag_gems/fused/fused_add_rms_norm.py:121-145).  Both tensors must be contiguous: they are updated where they lie."""
    logger.debug("GEMS FUSED_ADD_RMS_NORM FORWARD")
    rows, cols = _rows_of(x, normalized_shape)
    if not (x.is_contiguous() and residual.is_contiguous()):
        raise NotImplementedError("fused_add_rms_norm updates its operands in place and needs them contiguous")
    assert residual.shape == x.shape and residual.dtype == x.dtype
    if x.numel():
        _launch(x.view(rows, cols), residual.view(rows, cols), weight.contiguous(), eps, x.view(rows, cols), None, None, 0, 0.0,
                None, None, False)
    return x, residual


def rms_norm_per_token_group_quant_fp8(
    x: torch.Tensor,
    weight: torch.Tensor,
    group_size: int,
    eps: float = 1e-5,
    quant_eps: float = 1e-10,
    dtype: Optional[torch.dtype] = None,
    column_major_scales: bool = False,
    scale_ue8m0: bool = False,
    *,
    residual: Optional[torch.Tensor] = None,
    scale_rule: Optional[str] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``per_token_group_quant_fp8(rms_norm(x, (x.shape[-1],), weight, eps), group_size, quant_eps, ...)`` in one pass
    over x; with ``residual`` the norm is ``fused_add_rms_norm``'s and ``residual`` is updated in place (x is not).

    The normalised tensor is rounded to x's dtype as the separate kernel would store it, but never written.
    Same codes and scales, bit for bit, as the two calls.  Returns (x_q, x_s) shaped as per_token_group_quant_fp8's.
    """
    logger.debug("GEMS RMS_NORM PER TOKEN GROUP QUANT FP8")
    fp8_dtype = SUPPORTED_FP8_DTYPE if dtype is None else dtype
    cols = x.shape[-1]
    assert cols % group_size == 0, f"the last dimension of `x` {cols} must be divisible by `group_size` {group_size}"
    if fp8_dtype not in _FP8_DTYPES:
        raise NotImplementedError(f"rms_norm_per_token_group_quant_fp8: unsupported output dtype {fp8_dtype}")
    x = x.contiguous()
    if residual is not None:
        assert residual.shape == x.shape and residual.dtype == x.dtype
        if not residual.is_contiguous():
            raise NotImplementedError("the residual is updated in place and must be contiguous")
    x_q = torch.empty(x.shape, device=x.device, dtype=fp8_dtype)
    if column_major_scales:
        if x.dim() != 2:
            raise NotImplementedError("column_major_scales needs a 2-D input")
        x_s = torch.empty((cols // group_size, x.shape[0]), device=x.device, dtype=torch.float32).permute(-1, -2)
    else:
        x_s = torch.empty(x.shape[:-1] + (cols // group_size,), device=x.device, dtype=torch.float32)
    if x.numel() == 0:
        return x_q, x_s
    s2d = x_s if x_s.dim() == 2 else x_s.view(-1, x_s.shape[-1])
    _launch(x.view(-1, cols), residual.view(-1, cols) if residual is not None else None, weight.contiguous(), eps, None,
            x_q.view(-1, cols), s2d, group_size, quant_eps, fp8_dtype, scale_rule, scale_ue8m0)
    return x_q, x_s
