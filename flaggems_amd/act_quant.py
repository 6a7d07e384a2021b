"""Per-token-group activation quantizers (host side).

Mirrors the reference entry points
  act_quant_triton          src/flag_gems/fused/act_quant.py:111-174
  per_token_group_quant_fp8 src/flag_gems/ops/per_token_group_quant_fp8.py:227-336
and the vLLM op adapter     src/flag_gems/patches/patch_vllm_all.py:425-448
with the same parameters, defaults, return conventions and assertion behaviour.  The work is done
by the HIP kernel behind fg_group_quant_fp8.

Rounding contract.  Codes and scales are bit-identical to the reference's torch implementations
(tests/test_act_quant.py:48-98 for act_quant_triton, tests/test_per_token_group_quant_fp8.py:23-48
for per_token_group_quant_fp8): scale = amax * fp32(1/448); act_quant multiplies by the rounded
reciprocal of the scale, per_token_group_quant_fp8 divides; the eps floor of
per_token_group_quant_fp8 is applied in the input's dtype.  ``scale_rule="div"`` selects the
true-quotient scale amax / 448 that the reference's device kernel and MoE fallback use
(src/flag_gems/fused/fused_moe.py:664-668).
"""
from __future__ import annotations

import functools
import os
import logging
from typing import Optional, Tuple

import torch

from . import _lib

logger = logging.getLogger("flag_gems." + __name__.split(".")[-1])

# gfx950 converts to and from OCP e4m3fn natively
SUPPORTED_FP8_DTYPE = torch.float8_e4m3fn

_IN_DTYPES = (torch.bfloat16, torch.float16, torch.float32)
_FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2)


@functools.lru_cache(maxsize=64)
def _round_to_dtype(value: float, dtype: torch.dtype) -> float:
    return float(torch.tensor(value, dtype=dtype).float())


def _scale_rule_code(rule: Optional[str]) -> int:
    if rule is None or rule == "mul":
        return _lib.FG_SCALE_MUL_INV
    if rule == "div":
        return _lib.FG_SCALE_DIV
    raise ValueError(f"scale_rule must be 'mul' or 'div', got {rule!r}")


# Which of the reference's two formulations ``per_token_group_quant_fp8`` and the vLLM operator
# ``_C::per_token_group_fp8_quant`` follow when the caller does not say (they differ in the last bit of about half of
# all scales):
#   "test_reference": scale = amax * fp32(1/448) with the floor ``eps`` rounded to the input's dtype -- the torch
#                     helper the reference's unit test compares its kernel with
#                     (tests/test_per_token_group_quant_fp8.py:23-48);
#   "kernel":         scale = max(amax, eps) / 448 with ``eps`` as an fp32 value -- what the reference's device kernel
#                     computes (src/flag_gems/ops/per_token_group_quant_fp8.py:55-70).
# Process-wide; the environment variable FLAGGEMS_AMD_GROUP_QUANT_RULE sets the initial value.
_GROUP_QUANT_RULES = ("test_reference", "kernel")
_group_quant_rule = os.environ.get("FLAGGEMS_AMD_GROUP_QUANT_RULE", "test_reference")
if _group_quant_rule not in _GROUP_QUANT_RULES:
    raise ValueError(f"FLAGGEMS_AMD_GROUP_QUANT_RULE must be one of {_GROUP_QUANT_RULES}, got {_group_quant_rule!r}")


def set_group_quant_rule(rule: str) -> str:
    """Select the default formulation (see above); returns the previous one."""
    global _group_quant_rule
    if rule not in _GROUP_QUANT_RULES:
        raise ValueError(f"rule must be one of {_GROUP_QUANT_RULES}, got {rule!r}")
    previous, _group_quant_rule = _group_quant_rule, rule
    return previous


def get_group_quant_rule() -> str:
    return _group_quant_rule


def _default_rule_and_floor(eps: float, dtype: torch.dtype):
    if _group_quant_rule == "kernel":
        return _lib.FG_SCALE_DIV, _round_to_dtype(float(eps), torch.float32)
    return _lib.FG_SCALE_MUL_INV, _round_to_dtype(float(eps), dtype)


def _launch_group_quant(
    x2d: torch.Tensor,
    q2d: torch.Tensor,
    s2d: torch.Tensor,
    group_size: int,
    floor: float,
    fp8_min: float,
    fp8_max: float,
    scale_rule: int,
    quotient_rule: int,
    pow2_rule: int,
) -> None:
    """x2d [R, C] unit column stride; q2d same shape; s2d [R, C/g] any strides."""
    _lib.require_gpu(x2d, "group quantizer")
    rows, cols = x2d.shape
    with _lib.device_guard(x2d.device):
        status = _lib.fast().group_quant_fp8(
            _lib.address("fg_group_quant_fp8"),
            x2d.data_ptr(), _lib.DTYPE_CODE[x2d.dtype], rows, cols, x2d.stride(0) if rows > 1 else max(cols, x2d.stride(0)),
            q2d.data_ptr(), _lib.DTYPE_CODE[q2d.dtype], q2d.stride(0) if rows > 1 else max(cols, q2d.stride(0)),
            s2d.data_ptr(), s2d.stride(0), s2d.stride(1),
            group_size, floor, fp8_min, fp8_max, 1.0 / fp8_max,
            scale_rule, quotient_rule, pow2_rule,
            _lib.current_stream_ptr(x2d.device),
        )
    _lib.check(status, "fg_group_quant_fp8")


def act_quant_triton(
    x: torch.Tensor, block_size: int = 128, scale_fmt: Optional[str] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Block-wise FP8 quantization of the last dimension.

    Returns (y, s): y has x's shape and dtype float8_e4m3fn, s has shape
    ``x.shape[:-1] + (x.shape[-1] // block_size,)`` and dtype float32.  With ``scale_fmt`` set the
    scale is rounded up to a power of two.  The name is kept for drop-in compatibility; nothing
    here uses Triton.
    """
    logger.debug("GEMS ACT_QUANT")
    assert x.is_contiguous(), "Input tensor must be contiguous"
    assert (
        x.size(-1) % block_size == 0
    ), f"Last dimension size must be divisible by block_size (block_size={block_size})"
    if x.dtype not in _IN_DTYPES:
        raise NotImplementedError(f"act_quant: unsupported input dtype {x.dtype}")
    n = x.size(-1)
    n_blocks = n // block_size
    y = torch.empty_like(x, dtype=torch.float8_e4m3fn)
    s = x.new_empty(*x.size()[:-1], n_blocks, dtype=torch.float32)
    if x.numel() == 0:
        return y, s
    _launch_group_quant(
        x.view(-1, n), y.view(-1, n), s.view(-1, n_blocks), block_size,
        floor=1e-4, fp8_min=-448.0, fp8_max=448.0,
        scale_rule=_lib.FG_SCALE_MUL_INV, quotient_rule=_lib.FG_QUOT_RECIP_MUL,
        pow2_rule=_lib.FG_POW2_BITS if scale_fmt is not None else _lib.FG_POW2_NONE,
    )
    return y, s


def _as_rows(x: torch.Tensor) -> torch.Tensor:
    """View x as [rows, last] with unit column stride (copies only if the layout forces it)."""
    if x.dim() == 2:
        return x
    if x.dim() == 1:
        return x.view(1, -1)
    if not x.is_contiguous():
        x = x.contiguous()
    return x.view(-1, x.shape[-1])


def per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    dtype: Optional[torch.dtype] = None,
    column_major_scales: bool = False,
    scale_ue8m0: bool = False,
    *,
    scale_rule: Optional[str] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token-group quantization of ``x`` along its last dimension.

    Returns (x_q, x_s).  ``x_s`` is float32 of shape ``x.shape[:-1] + (x.shape[-1] // group_size,)``,
    row-major, or with strides (1, M) when ``column_major_scales`` is set.
    """
    logger.debug("GEMS PER TOKEN GROUP QUANT FP8")
    fp8_dtype = SUPPORTED_FP8_DTYPE if dtype is None else dtype
    assert x.shape[-1] % group_size == 0, (
        f"the last dimension of `x` {x.shape[-1]} must be divisible "
        f"by `group_size` {group_size}"
    )
    assert x.stride(-1) == 1, "`x` groups must be contiguous"
    if fp8_dtype not in _FP8_DTYPES:
        raise NotImplementedError(f"per_token_group_quant_fp8: unsupported output dtype {fp8_dtype}")
    if x.dtype not in _IN_DTYPES:
        raise NotImplementedError(f"per_token_group_quant_fp8: unsupported input dtype {x.dtype}")
    finfo = torch.finfo(fp8_dtype)

    # the reference kernel addresses x_q as a dense row-major image of x; allocate it that way
    x_q = torch.empty(x.shape, device=x.device, dtype=fp8_dtype)
    if column_major_scales:
        shape = (x.shape[-1] // group_size,) + x.shape[:-1]
        x_s = torch.empty(shape, device=x.device, dtype=torch.float32).permute(-1, -2)
    else:
        shape = x.shape[:-1] + (x.shape[-1] // group_size,)
        x_s = torch.empty(shape, device=x.device, dtype=torch.float32)
    if x.numel() == 0:
        return x_q, x_s

    x2d = _as_rows(x)
    q2d = x_q.view(-1, x.shape[-1])
    if x_s.dim() == 2:
        s2d = x_s
    elif not column_major_scales:
        s2d = x_s.view(-1, x_s.shape[-1])
    else:
        raise NotImplementedError("column_major_scales needs a 2-D input")
    if scale_rule is None:
        rule_code, floor = _default_rule_and_floor(eps, x.dtype)
    else:
        rule_code, floor = _scale_rule_code(scale_rule), _round_to_dtype(float(eps), x.dtype)
    _launch_group_quant(
        x2d, q2d, s2d, group_size,
        floor=floor, fp8_min=finfo.min, fp8_max=finfo.max,
        scale_rule=rule_code, quotient_rule=_lib.FG_QUOT_DIV,
        pow2_rule=_lib.FG_POW2_LOG2 if scale_ue8m0 else _lib.FG_POW2_NONE,
    )
    return x_q, x_s


def per_token_group_fp8_quant_into(
    input: torch.Tensor,
    output_q: torch.Tensor,
    output_s: torch.Tensor,
    group_size: int,
    eps: float,
    fp8_min: float,
    fp8_max: float,
    scale_ue8m0: bool = False,
) -> None:
    """vLLM ``_C::per_token_group_fp8_quant``: quantize into caller-owned buffers, honouring the
    strides of ``output_s`` (row- or column-major).  The reference adapter computes into fresh
    tensors and copies (src/flag_gems/patches/patch_vllm_all.py:425-448); here the kernel writes
    the caller's buffers directly."""
    logger.debug("GEMS PER TOKEN GROUP QUANT FP8")
    assert input.shape[-1] % group_size == 0
    assert input.stride(-1) == 1, "`x` groups must be contiguous"
    assert output_q.shape == input.shape and output_s.dtype == torch.float32
    if input.numel() == 0:
        return
    x2d = _as_rows(input)
    if output_q.stride(-1) != 1 or (output_q.dim() > 2 and not output_q.is_contiguous()):
        raise NotImplementedError("output_q must have unit stride in its last dimension")
    q2d = output_q if output_q.dim() == 2 else output_q.view(-1, input.shape[-1])
    s2d = output_s if output_s.dim() == 2 else output_s.view(-1, output_s.shape[-1])
    rule_code, floor = _default_rule_and_floor(eps, input.dtype)
    _launch_group_quant(
        x2d, q2d, s2d, group_size,
        floor=floor, fp8_min=float(fp8_min), fp8_max=float(fp8_max),
        scale_rule=rule_code, quotient_rule=_lib.FG_QUOT_DIV,
        pow2_rule=_lib.FG_POW2_LOG2 if scale_ue8m0 else _lib.FG_POW2_NONE,
    )


def per_block_cast_to_fp8(
    x: torch.Tensor, use_ue8m0: bool = True, gran_k: int = 128
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantize a 2-D weight to e4m3fn with one fp32 scale per ``gran_k x gran_k`` block.

    Same parameters, defaults and results (bit for bit) as the torch helper the reference builds its
    block-quantized weights with (tests/test_fp8_einsum.py:89-103, benchmark/test_fp8_einsum.py:82-96):
    blocks over the edge are padded with zeros, amax is floored at 1e-4, scale = amax / 448 (rounded up to
    a power of two when ``use_ue8m0``), codes = x * (1 / scale).  Returns (codes [m, n] contiguous,
    scales [ceil(m / gran_k), ceil(n / gran_k)] fp32).
    """
    logger.debug("GEMS PER_BLOCK_CAST_TO_FP8")
    assert x.dim() == 2
    if x.dtype not in _IN_DTYPES:
        raise NotImplementedError(f"per_block_cast_to_fp8: unsupported input dtype {x.dtype}")
    m, n = x.shape
    q = torch.empty((m, n), dtype=torch.float8_e4m3fn, device=x.device)
    sf = torch.empty((-(-m // gran_k), -(-n // gran_k)), dtype=torch.float32, device=x.device)
    if x.numel() == 0:
        return q, sf
    if x.stride(1) != 1:
        x = x.contiguous()
    _lib.require_gpu(x, "block quantizer")
    lib = _lib.load()
    with _lib.device_guard(x.device):
        status = lib.fg_block_quant_fp8(
            x.data_ptr(), _lib.DTYPE_CODE[x.dtype], m, n, x.stride(0) if m > 1 else max(n, x.stride(0)),
            q.data_ptr(), _lib.DTYPE_CODE[q.dtype], n,
            sf.data_ptr(), sf.stride(0), sf.stride(1),
            gran_k, gran_k, 1e-4, -448.0, 448.0, 1.0 / 448.0,
            _lib.FG_SCALE_DIV, _lib.FG_QUOT_RECIP_MUL, _lib.FG_POW2_BITS_CLAMPED if use_ue8m0 else _lib.FG_POW2_NONE,
            _lib.current_stream_ptr(x.device),
        )
    _lib.check(status, "fg_block_quant_fp8")
    return q, sf


def per_token_cast_to_fp8(
    x: torch.Tensor, use_ue8m0: bool = True, gran_k: int = 128
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantize a 2-D activation to e4m3fn with one fp32 scale per ``1 x gran_k`` group.

    Same parameters, defaults and results (bit for bit) as the torch helper of the reference's einsum test
    (tests/test_fp8_einsum.py:70-86): amax floored at 1e-4, scale = amax / 448 (rounded up to a power of two when
    ``use_ue8m0``), codes = x * (1 / scale).  The last dimension must be a multiple of ``gran_k`` (the reference
    pads with zeros otherwise; not implemented here).  Returns (codes [m, n], scales [m, n / gran_k] fp32).
    """
    logger.debug("GEMS PER_TOKEN_CAST_TO_FP8")
    assert x.dim() == 2
    if x.dtype not in _IN_DTYPES:
        raise NotImplementedError(f"per_token_cast_to_fp8: unsupported input dtype {x.dtype}")
    m, n = x.shape
    if n % gran_k != 0:
        raise NotImplementedError(f"per_token_cast_to_fp8: last dimension {n} is not a multiple of {gran_k}")
    if x.stride(1) != 1:
        x = x.contiguous()
    q = torch.empty((m, n), dtype=torch.float8_e4m3fn, device=x.device)
    sf = torch.empty((m, n // gran_k), dtype=torch.float32, device=x.device)
    if x.numel() == 0:
        return q, sf
    _launch_group_quant(
        x, q, sf, gran_k, floor=1e-4, fp8_min=-448.0, fp8_max=448.0,
        scale_rule=_lib.FG_SCALE_DIV, quotient_rule=_lib.FG_QUOT_RECIP_MUL,
        pow2_rule=_lib.FG_POW2_BITS_CLAMPED if use_ue8m0 else _lib.FG_POW2_NONE,
    )
    return q, sf


def silu_and_mul_packed(x: torch.Tensor) -> torch.Tensor:
    """``silu(x[..., :d]) * x[..., d:]`` with d = x.shape[-1] // 2, in x's dtype.

    The arithmetic of the reference's activation kernel (src/flag_gems/fused/silu_and_mul.py:13-18 and
    src/flag_gems/fused/fused_moe.py:795-800): fp32 ``g / (1 + exp(-g)) * u``, rounded once to the output type,
    applied to the gate and up halves of one tensor the way the expert layers hold them."""
    logger.debug("GEMS SILU_AND_MUL")
    assert x.shape[-1] % 2 == 0 and x.stride(-1) == 1
    if x.dtype not in _IN_DTYPES:
        raise NotImplementedError(f"silu_and_mul_packed: unsupported input dtype {x.dtype}")
    d = x.shape[-1] // 2
    out = torch.empty(x.shape[:-1] + (d,), dtype=x.dtype, device=x.device)
    return silu_and_mul_packed_out(out, x)


def silu_and_mul_packed_out(out: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """The same into ``out`` (x's shape with half the last dimension, contiguous): what vLLM's ``_C::silu_and_mul(out,
    input)`` asks for (src/flag_gems/patches/patch_vllm_all.py:276-279)."""
    assert x.shape[-1] % 2 == 0 and x.stride(-1) == 1
    if x.dtype not in _IN_DTYPES:
        raise NotImplementedError(f"silu_and_mul_packed: unsupported input dtype {x.dtype}")
    d = x.shape[-1] // 2
    assert out.shape == x.shape[:-1] + (d,) and out.dtype == x.dtype and out.device == x.device and out.is_contiguous()
    if out.numel() == 0:
        return out
    x2d = _as_rows(x)
    _lib.require_gpu(x2d, "silu_and_mul")
    rows = x2d.shape[0]
    with _lib.device_guard(x.device):
        status = _lib.load().fg_silu_mul(
            x2d.data_ptr(), _lib.DTYPE_CODE[x.dtype], rows, d, x2d.stride(0) if rows > 1 else max(2 * d, x2d.stride(0)), d,
            out.data_ptr(), d, _lib.current_stream_ptr(x.device))
    _lib.check(status, "fg_silu_mul")
    return out


def silu_and_mul_per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    dtype: Optional[torch.dtype] = None,
    column_major_scales: bool = False,
    scale_ue8m0: bool = False,
    *,
    scale_rule: Optional[str] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``per_token_group_quant_fp8(silu_and_mul_packed(x), group_size, ...)`` in one pass over x.

    The step between the two GEMMs of an expert or MLP layer (src/flag_gems/fused/fused_moe.py:2108-2122): the
    activated tensor is rounded to x's dtype as the separate kernel would store it, but never written.
    Same codes and scales, bit for bit, as the two calls.  x [..., 2 d]; returns (x_q [..., d], x_s [..., d / group_size]).
    """
    logger.debug("GEMS SILU_AND_MUL PER TOKEN GROUP QUANT FP8")
    fp8_dtype = SUPPORTED_FP8_DTYPE if dtype is None else dtype
    assert x.shape[-1] % 2 == 0 and x.stride(-1) == 1
    d = x.shape[-1] // 2
    assert d % group_size == 0, f"half of the last dimension of `x` {d} must be divisible by `group_size` {group_size}"
    if fp8_dtype not in _FP8_DTYPES:
        raise NotImplementedError(f"silu_and_mul_per_token_group_quant_fp8: unsupported output dtype {fp8_dtype}")
    if x.dtype not in _IN_DTYPES:
        raise NotImplementedError(f"silu_and_mul_per_token_group_quant_fp8: unsupported input dtype {x.dtype}")
    finfo = torch.finfo(fp8_dtype)
    lead = x.shape[:-1]
    x_q = torch.empty(lead + (d,), device=x.device, dtype=fp8_dtype)
    if column_major_scales:
        if x.dim() != 2:
            raise NotImplementedError("column_major_scales needs a 2-D input")
        x_s = torch.empty((d // group_size, x.shape[0]), device=x.device, dtype=torch.float32).permute(-1, -2)
    else:
        x_s = torch.empty(lead + (d // group_size,), device=x.device, dtype=torch.float32)
    if x_q.numel() == 0:
        return x_q, x_s
    x2d = _as_rows(x)
    _lib.require_gpu(x2d, "fused activation + quantizer")
    rows = x2d.shape[0]
    q2d = x_q.view(-1, d)
    s2d = x_s if x_s.dim() == 2 else x_s.view(-1, x_s.shape[-1])
    if scale_rule is None:  # the process-wide default, as in per_token_group_quant_fp8: the fused call stays its twin
        rule_code, floor = _default_rule_and_floor(eps, x.dtype)
    else:
        rule_code, floor = _scale_rule_code(scale_rule), _round_to_dtype(float(eps), x.dtype)
    with _lib.device_guard(x.device):
        status = _lib.load().fg_silu_mul_group_quant_fp8(
            x2d.data_ptr(), _lib.DTYPE_CODE[x.dtype], rows, d, x2d.stride(0) if rows > 1 else max(2 * d, x2d.stride(0)), d,
            q2d.data_ptr(), _lib.DTYPE_CODE[fp8_dtype], d,
            s2d.data_ptr(), s2d.stride(0), s2d.stride(1),
            group_size, floor, finfo.min, finfo.max, 1.0 / finfo.max,
            rule_code, _lib.FG_QUOT_DIV, _lib.FG_POW2_LOG2 if scale_ue8m0 else _lib.FG_POW2_NONE,
            _lib.current_stream_ptr(x.device))
    _lib.check(status, "fg_silu_mul_group_quant_fp8")
    return x_q, x_s
