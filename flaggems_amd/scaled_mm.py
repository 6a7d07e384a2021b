"""aten::_scaled_mm / aten::_scaled_mm.out (host side).

Mirrors src/flag_gems/ops/scaled_mm.py:214-273 (argument normalisation and RuntimeError messages)
and :333-452 (entry points) of the reference.  FP8 (e4m3fn) and int8 operands run on the HIP scaled
GEMMs (the reference sends both to cutlass_scaled_mm, :289-316); bf16, fp16 and fp32 operands run on the
generic HIP kernel that stands in for the reference's Triton scaled_mm_kernel (:37-133, :365-422).
"""
from __future__ import annotations

import logging

import torch

from .cutlass_scaled_mm import _launch_scaled_gemm, _launch_scaled_generic_gemm, _launch_scaled_int8_gemm

logger = logging.getLogger("flag_gems." + __name__.split(".")[-1])

def _scale_vector(scale, count, name, matrix_shape):
    """One scale (any tensor with a single element) or `count` of them, given as ``[count]`` or as the
    matrix-shaped column / row ``matrix_shape``; returned as a contiguous 1-D tensor.  The launchers tell the two
    kinds apart by the element count.  Error text: src/flag_gems/ops/scaled_mm.py:245-249."""
    if scale.numel() != 1 and tuple(scale.shape) not in ((count,), matrix_shape):
        raise RuntimeError(
            f"{name} must be a scalar tensor or have shape ({matrix_shape[0]}, {matrix_shape[1]})"
        )
    return scale.reshape(-1).contiguous()


def _scaled_mm_impl(self, mat2, scale_a, scale_b, bias, out_dtype, out):
    # argument errors in the reference's order and wording (src/flag_gems/ops/scaled_mm.py:214-273, 350-351)
    for name, operand in (("self", self), ("mat2", mat2)):
        if operand.dim() != 2:
            raise RuntimeError(f"{name} must be a matrix")
    (M, K), (K2, N) = self.shape, mat2.shape
    if K != K2:
        raise RuntimeError(f"mat1 and mat2 shapes cannot be multiplied ({M}x{K} and {K2}x{N})")
    if self.dtype != mat2.dtype:
        raise RuntimeError(f"self and mat2 must have the same dtype, but got {self.dtype} and {mat2.dtype}")
    # result type: the explicit out_dtype, else that of the tensor to fill, else the operands'
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype if out_dtype is not None else self.dtype, device=self.device)
    else:
        if out_dtype is not None and out.dtype != out_dtype:
            raise RuntimeError("out_dtype must be the same as the dtype of the provided out tensor")
        if tuple(out.shape) != (M, N):
            raise RuntimeError("Incompatible output shape")
    scale_a = _scale_vector(scale_a, M, "scale_a", (M, 1))
    scale_b = _scale_vector(scale_b, N, "scale_b", (1, N))
    if bias is not None:
        if bias.numel() != N:
            raise RuntimeError(f"Bias must be size {N} but got {bias.numel()}")
        bias = bias.reshape(N).contiguous()
    if M == 0 or N == 0:
        return out

    generic = self.dtype in (torch.bfloat16, torch.float16, torch.float32)
    if not generic and self.dtype not in (torch.float8_e4m3fn, torch.int8):
        raise NotImplementedError(
            f"_scaled_mm: operands must be float8_e4m3fn, int8, bfloat16, float16 or float32 in the gfx950 build, got {self.dtype}"
        )
    if (self.dtype == torch.int8 or generic) and out.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise NotImplementedError(f"_scaled_mm: {self.dtype} operands need a bf16, fp16 or fp32 out_dtype, got {out.dtype}")
    if bias is not None and bias.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise NotImplementedError(f"_scaled_mm: unsupported bias dtype {bias.dtype}")
    if scale_a.dtype != torch.float32 or scale_b.dtype != torch.float32:
        scale_a, scale_b = scale_a.to(torch.float32), scale_b.to(torch.float32)
    # the kernels want K-contiguous rows on both sides: self row-major, mat2 column-major
    if self.stride(1) != 1:
        self = self.contiguous()
    if mat2.stride(0) != 1:
        mat2 = mat2.t().contiguous().t()
    if generic and K == 0:  # empty sums: zeros (plus the bias), no kernel
        out.zero_()
        if bias is not None:
            out.add_(bias.to(torch.float32).reshape(1, N).to(out.dtype))
        return out
    if generic:
        # 16-byte loads along K: pad K with zeros (they add nothing to the sums) and realign rows where needed
        per_load = 16 // self.element_size()
        if K % per_load != 0:
            pad = per_load - K % per_load
            self = torch.nn.functional.pad(self, (0, pad))
            mat2 = torch.nn.functional.pad(mat2.t(), (0, pad)).t()
        if self.data_ptr() % 16 != 0 or (M > 1 and (self.stride(0) * self.element_size()) % 16 != 0):
            self = self.clone(memory_format=torch.contiguous_format)
        if mat2.data_ptr() % 16 != 0 or (N > 1 and (mat2.stride(1) * mat2.element_size()) % 16 != 0):
            mat2 = mat2.t().clone(memory_format=torch.contiguous_format).t()
    target = out if out.stride(1) == 1 else torch.empty((M, N), dtype=out.dtype, device=out.device)
    if generic:
        _launch_scaled_generic_gemm(target, self, mat2, scale_a, scale_b, bias)
    elif self.dtype == torch.int8:
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
