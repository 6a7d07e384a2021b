"""Batched block-scaled FP8 GEMM and the einsum built on it (host side).

Mirrors the reference entry points
  w8a8_block_fp8_bmm  src/flag_gems/runtime/backend/_nvidia/hopper/ops/w8a8_block_fp8_bmm.py:629-779
  fp8_einsum          src/flag_gems/runtime/backend/_nvidia/hopper/ops/fp8_einsum.py:22-68
with the same parameters, defaults and assertions.  The reference ships them for one vendor back-end only;
here they run on the kernels of w8a8_block_fp8_matmul, one launch per batch entry.
"""
from __future__ import annotations

import logging
from typing import List, Optional

import torch

from . import _lib

logger = logging.getLogger("flag_gems." + __name__.split(".")[-1])

_OUT_DTYPES = (torch.bfloat16, torch.float16, torch.float32)


def w8a8_block_fp8_bmm(
    x: torch.Tensor,
    y: torch.Tensor,
    xs: torch.Tensor,
    ys: torch.Tensor,
    block_size: List[int] = [128, 128],
    z: Optional[torch.Tensor] = None,
    output_dtype: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """z[i] = block_fp8_matmul(x[i], y[i]) for every batch entry i.

    x [B, M, K] e4m3fn, y [B, N, K] e4m3fn (unit stride in K, any other strides), xs [B, M, K/128] fp32 with any
    strides, ys [B, N/128, K/128] fp32, z [B, M, N] (allocated when None; unit stride in N)."""
    logger.debug("GEMS W8A8_BLOCK_FP8_BMM")
    assert len(block_size) == 2
    block_n, block_k = block_size
    assert block_n == 128 and block_k == 128, "this kernel assumes 128x128 block-wise FP8 scales"
    assert x.ndim == 3 and y.ndim == 3 and xs.ndim == 3 and ys.ndim == 3
    assert x.shape[0] == y.shape[0] == xs.shape[0] == ys.shape[0]
    assert x.shape[-1] == y.shape[-1]
    assert x.shape[:-1] == xs.shape[:-1]
    assert x.stride(-1) == 1 and y.stride(-1) == 1
    B, M, K = x.shape
    _, N, _ = y.shape
    assert K % block_k == 0 and N % block_n == 0
    assert xs.shape[-1] == K // block_k and ys.shape == (B, N // block_n, K // block_k)
    if z is None:
        z = torch.empty((B, M, N), device=x.device, dtype=output_dtype)
    else:
        assert z.shape == (B, M, N) and z.device == x.device and z.dtype == output_dtype
        assert z.stride(-1) == 1
    if x.dtype != torch.float8_e4m3fn or y.dtype != torch.float8_e4m3fn:
        raise NotImplementedError(f"w8a8_block_fp8_bmm: operands must be float8_e4m3fn, got {x.dtype}, {y.dtype}")
    if output_dtype not in _OUT_DTYPES:
        raise NotImplementedError(f"w8a8_block_fp8_bmm: unsupported output dtype {output_dtype}")
    if xs.dtype != torch.float32 or ys.dtype != torch.float32:
        xs, ys = xs.to(torch.float32), ys.to(torch.float32)
    if B == 0 or M == 0 or N == 0:
        return z
    _lib.require_gpu(x, "batched block fp8 gemm")
    lib = _lib.load()
    dev = x.device
    with _lib.device_guard(dev):
        ws_bytes = _lib.cached_workspace_bytes("fg_batched_block_fp8_gemm_workspace_bytes", B, M, N, K)
        ws = _lib.workspace(dev, ws_bytes) if ws_bytes else None
        status = lib.fg_batched_block_fp8_gemm(
            x.data_ptr(), x.stride(1) if M > 1 else max(K, x.stride(1)), x.stride(0),
            y.data_ptr(), y.stride(1) if N > 1 else max(K, y.stride(1)), y.stride(0),
            xs.data_ptr(), xs.stride(1), xs.stride(2), xs.stride(0),
            ys.data_ptr(), ys.stride(1), ys.stride(2), ys.stride(0),
            z.data_ptr(), z.stride(1) if M > 1 else max(N, z.stride(1)), z.stride(0), _lib.DTYPE_CODE[z.dtype],
            B, M, N, K, block_n, block_k,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            _lib.current_stream_ptr(dev),
        )
    _lib.check(status, "fg_batched_block_fp8_gemm")
    return z


def fp8_einsum(
    equation: str,
    x: torch.Tensor,
    xs: torch.Tensor,
    y: torch.Tensor,
    ys: torch.Tensor,
    block_size: List[int] = [128, 128],
    output_dtype: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """Block-wise FP8 einsum; only ``"bhr,hdr->bhd"``: out[b,h,d] = sum_r x[b,h,r] * y[h,d,r].

    x (b, h, r) e4m3fn with xs (b, h, r // block_k) per-token scales, y (h, d, r) e4m3fn with
    ys (h, d // block_n, r // block_k) block scales; returns a new (b, h, d) tensor."""
    logger.debug("GEMS FP8_EINSUM")
    assert equation == "bhr,hdr->bhd", f"fp8_einsum only supports 'bhr,hdr->bhd', got {equation!r}"
    b, h, r = x.shape
    h2, d, r2 = y.shape
    assert h2 == h and r2 == r, f"x {tuple(x.shape)} / y {tuple(y.shape)} mismatch"
    z = torch.empty((b, h, d), device=x.device, dtype=output_dtype)
    # h is the batch dimension; the permutes are views (r stays contiguous) and the strides go to the kernels
    w8a8_block_fp8_bmm(x.permute(1, 0, 2), y, xs.permute(1, 0, 2), ys, block_size=block_size,
                       z=z.permute(1, 0, 2), output_dtype=output_dtype)
    return z
