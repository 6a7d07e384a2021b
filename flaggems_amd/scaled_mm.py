"""aten::_scaled_mm / aten::_scaled_mm.out (host side).

Mirrors src/flag_gems/ops/scaled_mm.py:214-273 (argument normalisation and RuntimeError messages)
and :333-452 (entry points) of the reference.  FP8 (e4m3fn) and int8 operands run on the HIP scaled
GEMMs (the reference sends both to cutlass_scaled_mm, :289-316); its generic Triton kernel for other
operand types is not part of this build and such calls raise NotImplementedError.
"""
from __future__ import annotations

import logging

import torch

from .cutlass_scaled_mm import _launch_scaled_gemm, _launch_scaled_int8_gemm

logger = logging.getLogger("flag_gems." + __name__.split(".")[-1])

SCALAR_SCALE = 0
VECTOR_SCALE = 1


def _resolve_out_dtype(self, out_dtype, out=None):
    if out_dtype is not None:
        if out is not None and out.dtype != out_dtype:
            raise RuntimeError("out_dtype must be the same as the dtype of the provided out tensor")
        return out_dtype
    if out is not None:
        return out.dtype
    return self.dtype


def _normalize_scale(scale, expected_size, *, is_left_scale):
    if scale.numel() == 1:
        return scale.reshape(1).contiguous(), SCALAR_SCALE
    valid = scale.ndim == 1 and scale.shape[0] == expected_size
    if is_left_scale:
        valid = valid or (scale.ndim == 2 and tuple(scale.shape) == (expected_size, 1))
    else:
        valid = valid or (scale.ndim == 2 and tuple(scale.shape) == (1, expected_size))
    if valid:
        return scale.reshape(expected_size).contiguous(), VECTOR_SCALE
    name = "scale_a" if is_left_scale else "scale_b"
    shape = f"({expected_size}, 1)" if is_left_scale else f"(1, {expected_size})"
    raise RuntimeError(f"{name} must be a scalar tensor or have shape {shape}")


def _normalize_bias(bias, cols):
    if bias is None:
        return None
    if bias.numel() != cols:
        raise RuntimeError(f"Bias must be size {cols} but got {bias.numel()}")
    return bias.reshape(cols).contiguous()


def _check_inputs(self, mat2):
    if self.ndim != 2:
        raise RuntimeError("self must be a matrix")
    if mat2.ndim != 2:
        raise RuntimeError("mat2 must be a matrix")
    if self.shape[1] != mat2.shape[0]:
        raise RuntimeError(
            f"mat1 and mat2 shapes cannot be multiplied ({self.shape[0]}x{self.shape[1]} "
            f"and {mat2.shape[0]}x{mat2.shape[1]})"
        )
    if self.dtype != mat2.dtype:
        raise RuntimeError(f"self and mat2 must have the same dtype, but got {self.dtype} and {mat2.dtype}")


def _scaled_mm_impl(self, mat2, scale_a, scale_b, bias, out_dtype, out):
    _check_inputs(self, mat2)
    M, K = self.shape
    _, N = mat2.shape
    output_dtype = _resolve_out_dtype(self, out_dtype, out)
    if out is None:
        out = torch.empty((M, N), dtype=output_dtype, device=self.device)
    elif tuple(out.shape) != (M, N):
        raise RuntimeError("Incompatible output shape")

    scale_a, _ = _normalize_scale(scale_a, M, is_left_scale=True)
    scale_b, _ = _normalize_scale(scale_b, N, is_left_scale=False)
    bias = _normalize_bias(bias, N)
    if M == 0 or N == 0:
        return out

    if self.dtype not in (torch.float8_e4m3fn, torch.int8):
        raise NotImplementedError(
            f"_scaled_mm: only float8_e4m3fn and int8 operands are implemented in the gfx950 build, got {self.dtype}"
        )
    if self.dtype == torch.int8 and out.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise NotImplementedError(f"_scaled_mm: int8 operands need a floating-point out_dtype, got {out.dtype}")
    if scale_a.dtype != torch.float32 or scale_b.dtype != torch.float32:
        scale_a, scale_b = scale_a.to(torch.float32), scale_b.to(torch.float32)
    # the kernel wants K-contiguous rows on both sides: self row-major, mat2 column-major
    if self.stride(1) != 1:
        self = self.contiguous()
    if mat2.stride(0) != 1:
        mat2 = mat2.t().contiguous().t()
    target = out if out.stride(1) == 1 else torch.empty((M, N), dtype=out.dtype, device=out.device)
    if self.dtype == torch.int8:
        _launch_scaled_int8_gemm(target, self, mat2, scale_a, scale_b, bias)
    else:
        _launch_scaled_gemm(target, self, mat2, scale_a, scale_b, bias)
    if target is not out:
        out.copy_(target)
    return out


def scaled_mm(self, mat2, scale_a, scale_b, bias=None, scale_result=None, out_dtype=None, use_fast_accum=False):
    """``scale_result`` and ``use_fast_accum`` are accepted and ignored, as in the reference."""
    logger.debug("GEMS SCALED_MM")
    return _scaled_mm_impl(self, mat2, scale_a, scale_b, bias, out_dtype, None)


def scaled_mm_out(
    self, mat2, scale_a, scale_b, bias=None, scale_result=None, out_dtype=None, use_fast_accum=False, *, out
):
    logger.debug("GEMS SCALED_MM_OUT")
    return _scaled_mm_impl(self, mat2, scale_a, scale_b, bias, out_dtype, out)
