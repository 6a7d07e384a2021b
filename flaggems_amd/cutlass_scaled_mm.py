"""cutlass_scaled_mm (host side): per-tensor / per-token x per-channel scaled FP8 or int8 GEMM with optional
bias, and the 128-block-wise FP8 variant, written into a caller-owned output.

Mirrors src/flag_gems/fused/cutlass_scaled_mm.py:371-431 (dispatch) and :475-526 (entry point) of
the reference: same argument order, same assertions and messages, returns None.  The reference
switches on the CUDA SM version read at import; this build targets gfx950 only, which PyTorch-ROCm
reports as capability (9, 5), i.e. the reference's "sm90" branch.
"""
from __future__ import annotations

import logging
from typing import Optional

import torch

from . import _lib
from .w8a8_block_fp8_matmul import _cdiv, _launch_block_gemm

logger = logging.getLogger("flag_gems." + __name__.split(".")[-1])

SCALE_BLOCK_K, SCALE_BLOCK_N = 128, 128


def get_sm_version_num() -> int:
    """gfx950 under PyTorch-ROCm reports device capability (9, 5); no device is probed here."""
    return 95


SM_VERSION_NUM = get_sm_version_num()


def _launch_scaled_gemm(c, a, b, a_scale, b_scale, bias) -> None:
    _lib.require_gpu(a, "scaled fp8 gemm")
    m, k = a.shape
    n = b.shape[1]
    dev = a.device
    with _lib.device_guard(dev):
        ws_bytes = _lib.cached_workspace_bytes("fg_scaled_fp8_gemm_workspace_bytes", m, n, k)
        ws = _lib.workspace(dev, ws_bytes) if ws_bytes else None
        status = _lib.fast().scaled_gemm(
            _lib.address("fg_scaled_fp8_gemm"),
            a.data_ptr(), a.stride(0) if m > 1 else max(k, a.stride(0)),
            b.data_ptr(), b.stride(1) if n > 1 else max(k, b.stride(1)),
            a_scale.data_ptr(), 1 if a_scale.numel() > 1 or m == 1 else 0,
            b_scale.data_ptr(), 1 if b_scale.numel() > 1 or n == 1 else 0,
            bias.data_ptr() if bias is not None else None,
            _lib.DTYPE_CODE[bias.dtype] if bias is not None else _lib.FG_BF16,
            c.data_ptr(), c.stride(0) if m > 1 else max(n, c.stride(0)), _lib.DTYPE_CODE[c.dtype],
            m, n, k,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            _lib.current_stream_ptr(dev),
        )
    _lib.check(status, "fg_scaled_fp8_gemm")


def _launch_scaled_int8_gemm(c, a, b, a_scale, b_scale, bias) -> None:
    _lib.require_gpu(a, "scaled int8 gemm")
    m, k = a.shape
    n = b.shape[1]
    dev = a.device
    with _lib.device_guard(dev):
        ws_bytes = _lib.cached_workspace_bytes("fg_scaled_int8_gemm_workspace_bytes", m, n, k)
        ws = _lib.workspace(dev, ws_bytes) if ws_bytes else None
        status = _lib.fast().scaled_gemm(
            _lib.address("fg_scaled_int8_gemm"),
            a.data_ptr(), a.stride(0) if m > 1 else max(k, a.stride(0)),
            b.data_ptr(), b.stride(1) if n > 1 else max(k, b.stride(1)),
            a_scale.data_ptr(), 1 if a_scale.numel() > 1 or m == 1 else 0,
            b_scale.data_ptr(), 1 if b_scale.numel() > 1 or n == 1 else 0,
            bias.data_ptr() if bias is not None else None,
            _lib.DTYPE_CODE[bias.dtype] if bias is not None else _lib.FG_BF16,
            c.data_ptr(), c.stride(0) if m > 1 else max(n, c.stride(0)), _lib.DTYPE_CODE[c.dtype],
            m, n, k,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            _lib.current_stream_ptr(dev),
        )
    _lib.check(status, "fg_scaled_int8_gemm")


def _launch_scaled_generic_gemm(c, a, b, a_scale, b_scale, bias) -> None:
    """bf16 / fp16 / fp32 operands: a [M, K] with unit column stride, b [K, N] with unit row stride (column-major)."""
    _lib.require_gpu(a, "scaled gemm")
    lib = _lib.load()
    m, k = a.shape
    n = b.shape[1]
    dev = a.device
    with _lib.device_guard(dev):
        status = lib.fg_scaled_gemm(
            a.data_ptr(), a.stride(0) if m > 1 else max(k, a.stride(0)),
            b.data_ptr(), b.stride(1) if n > 1 else max(k, b.stride(1)), _lib.DTYPE_CODE[a.dtype],
            a_scale.data_ptr(), 1 if a_scale.numel() > 1 or m == 1 else 0,
            b_scale.data_ptr(), 1 if b_scale.numel() > 1 or n == 1 else 0,
            bias.data_ptr() if bias is not None else None,
            _lib.DTYPE_CODE[bias.dtype] if bias is not None else _lib.FG_BF16,
            c.data_ptr(), c.stride(0) if m > 1 else max(n, c.stride(0)), _lib.DTYPE_CODE[c.dtype],
            m, n, k, _lib.current_stream_ptr(dev),
        )
    _lib.check(status, "fg_scaled_gemm")


def dispatch_scaled_mm(c, a, b, a_scale, b_scale, bias) -> None:
    assert a_scale.dtype == torch.float32, "a_scale must be float32"
    assert b_scale.dtype == torch.float32, "b_scale must be float32"

    if (a_scale.numel() == 1 or a_scale.numel() == a.size(0)) and (
        b_scale.numel() == 1 or b_scale.numel() == b.size(1)
    ):
        assert a_scale.is_contiguous(), "a_scale must be contiguous"
        assert b_scale.is_contiguous(), "b_scale must be contiguous"
        if a.dtype == torch.float8_e4m3fn:
            if c.dtype not in _lib.DTYPE_CODE or c.dtype == torch.float8_e5m2:
                raise NotImplementedError(f"cutlass_scaled_mm: unsupported output dtype {c.dtype}")
            if bias is not None and bias.dtype not in (torch.bfloat16, torch.float16, torch.float32):
                raise NotImplementedError(f"cutlass_scaled_mm: unsupported bias dtype {bias.dtype}")
            _launch_scaled_gemm(c, a, b, a_scale, b_scale, bias)
        else:
            assert a.dtype == torch.int8, f"Unsupported dtype: {a.dtype}"
            if c.dtype not in (torch.bfloat16, torch.float16, torch.float32):
                raise NotImplementedError(f"cutlass_scaled_mm (int8): unsupported output dtype {c.dtype}")
            if bias is not None and bias.dtype not in (torch.bfloat16, torch.float16, torch.float32):
                raise NotImplementedError(f"cutlass_scaled_mm: unsupported bias dtype {bias.dtype}")
            if b.dtype != torch.int8:
                raise NotImplementedError(f"cutlass_scaled_mm (int8): b is {b.dtype}")
            _launch_scaled_int8_gemm(c, a, b, a_scale, b_scale, bias)
    else:
        assert a_scale.dim() == 2, "a_scale must be 2D tensor for blockwise scaling"
        assert b_scale.dim() == 2, "b_scale must be 2D tensor for blockwise scaling"
        assert a.size(0) == a_scale.size(0), (
            f"a_scale must have same first dimension as a: "
            f"a.shape[0]={a.size(0)}, a_scale.shape[0]={a_scale.size(0)}"
        )
        assert _cdiv(a.size(1), 128) == a_scale.size(1), (
            f"a_scale second dimension mismatch: "
            f"triton.cdiv({a.size(1)}, 128)={_cdiv(a.size(1), 128)} != "
            f"a_scale.shape[1]={a_scale.size(1)}"
        )
        assert _cdiv(b.size(0), 128) == b_scale.size(0), (
            f"b_scale first dimension mismatch: "
            f"triton.cdiv({b.size(0)}, 128)={_cdiv(b.size(0), 128)} != "
            f"b_scale.shape[0]={b_scale.size(0)}"
        )
        assert _cdiv(b.size(1), 128) == b_scale.size(1), (
            f"b_scale second dimension mismatch: "
            f"triton.cdiv({b.size(1)}, 128)={_cdiv(b.size(1), 128)} != "
            f"b_scale.shape[1]={b_scale.size(1)}"
        )
        assert bias is None, "Bias not yet supported for blockwise scaled_mm"
        if a.dtype != torch.float8_e4m3fn:
            raise NotImplementedError(f"cutlass_scaled_mm (block-wise): unsupported dtype {a.dtype}")
        if c.dtype not in (torch.bfloat16, torch.float16, torch.float32):
            raise NotImplementedError(f"cutlass_scaled_mm (block-wise): unsupported output dtype {c.dtype}")
        # b is [K, N] column-major = N rows of K bytes; b_scale is [K/128, N/128]
        _launch_block_gemm(a, b.t(), a_scale, b_scale.t(), c, SCALE_BLOCK_N, SCALE_BLOCK_K)


def cutlass_scaled_mm(
    c: torch.Tensor,
    a: torch.Tensor,
    b: torch.Tensor,
    a_scale: torch.Tensor,
    b_scale: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
) -> None:
    logger.debug("GEMS CUTLASS SCALED MM")
    assert (
        a.dim() == 2 and b.dim() == 2 and c.dim() == 2
    ), "All inputs must be 2D tensors"
    assert c.size(0) == a.size(0), "Number of rows in c must equal number of rows in a"
    assert a.size(1) == b.size(0), "Number of columns in a must equal number of rows in b"
    assert b.size(1) == c.size(1), "Number of columns in b must equal number of columns in c"
    assert a.stride(1) == 1 and c.stride(1) == 1, "a and c must be row-major"
    assert b.stride(0) == 1, "b must be column-major"
    assert c.stride(0) % 16 == 0, "Row stride of c must be 16-byte aligned"
    assert b.stride(1) % 16 == 0, "Column stride of b must be 16-byte aligned"
    if bias is not None:
        assert bias.numel() == b.size(1), (
            f"Bias size {bias.numel()} must equal number of columns in b {b.size(1)}"
        )
        assert bias.is_contiguous(), "Bias must be contiguous"
        assert bias.dim() == 1, "Bias must be a 1D tensor"
    if c.numel() == 0:
        return None
    dispatch_scaled_mm(c, a, b, a_scale, b_scale, bias)
    return None
