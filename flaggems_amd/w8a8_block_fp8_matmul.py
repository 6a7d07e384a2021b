"""Block-scaled FP8 GEMM (host side).

Mirrors the reference entry points
  w8a8_block_fp8_matmul  src/flag_gems/ops/w8a8_block_fp8_matmul.py:173-232
  fp8_matmul             src/flag_gems/ops/fp8_matmul.py:137-205
  fp8_matmul_noop        cpp/lib/fp8_matmul.cpp:104-125 (checks and allocation only: a probe of the host overhead)
with the same parameters, defaults and assertions.  The reference picks a Triton tile from a
per-device YAML table; here the C library picks the HIP kernel variant from (M, N, K).
"""
from __future__ import annotations

import logging
import math
from typing import List

import torch

from . import _lib

logger = logging.getLogger("flag_gems." + __name__.split(".")[-1])

GROUP_SIZE = 128  # scale granularity of fp8_matmul (reference src/flag_gems/ops/fp8_matmul.py:42)
_OUT_DTYPES = (torch.bfloat16, torch.float16, torch.float32)


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def _launch_raw(dev, a_ptr, lda, b_ptr, ldb, as_ptr, as_rs, as_cs, bs_ptr, bs_rs, bs_cs, c_ptr, ldc, c_code, m, n, k,
                block_n: int, block_k: int, scales_pow2: bool) -> None:
    """The C-ABI call with everything already reduced to addresses and integers (decode-sized calls are host-bound:
    every tensor method that is not needed per call is kept out of this path)."""
    with _lib.device_guard(dev):
        stream = _lib.current_stream_ptr(dev)
        ws_bytes = _lib.cached_workspace_bytes("fg_block_fp8_gemm_workspace_bytes", m, n, k)
        if ws_bytes:
            ws = _lib.workspace(dev, ws_bytes, stream)
            ws_ptr, ws_len = ws.data_ptr(), ws.numel()
        else:
            ws_ptr, ws_len = None, 0
        status = _lib.fast().block_fp8_gemm(
            _lib.address("fg_block_fp8_gemm_pow2_scales" if scales_pow2 else "fg_block_fp8_gemm"),
            a_ptr, lda, b_ptr, ldb, as_ptr, as_rs, as_cs, bs_ptr, bs_rs, bs_cs, c_ptr, ldc, c_code,
            m, n, k, block_n, block_k, ws_ptr, ws_len, stream,
        )
    if status:
        _lib.check(status, "fg_block_fp8_gemm")


def _launch_block_gemm(a2d, b, as2d, bs, c2d, block_n: int, block_k: int, scales_pow2: bool = False) -> None:
    dev = a2d.device
    if dev.type != "cuda":
        _lib.require_gpu(a2d, "block fp8 gemm")
    m, k = a2d.shape
    n = b.shape[0]
    _launch_raw(
        dev,
        a2d.data_ptr(), a2d.stride(0) if m > 1 else max(k, a2d.stride(0)),
        b.data_ptr(), b.stride(0) if n > 1 else max(k, b.stride(0)),
        as2d.data_ptr(), as2d.stride(0), as2d.stride(1),
        bs.data_ptr(), bs.stride(0), bs.stride(1),
        c2d.data_ptr(), c2d.stride(0) if m > 1 else max(n, c2d.stride(0)), _lib.DTYPE_CODE[c2d.dtype],
        m, n, k, block_n, block_k, scales_pow2,
    )


def w8a8_block_fp8_matmul(
    A: torch.Tensor,
    B: torch.Tensor,
    As: torch.Tensor,
    Bs: torch.Tensor,
    block_size: List[int],
    output_dtype: torch.dtype = torch.bfloat16,
    scales_are_powers_of_two: bool = False,
) -> torch.Tensor:
    """C = (A dequantised by As per 1 x block_k group) @ (B dequantised by Bs per block_n x block_k block)^T.

    A [..., K] contiguous e4m3fn, As [..., ceil(K/block_k)] fp32, B [N, K] e4m3fn,
    Bs [ceil(N/block_n), ceil(K/block_k)] fp32; returns [..., N] in ``output_dtype``.

    ``scales_are_powers_of_two`` (not in the reference's signature): the caller's promise that every entry of As and
    Bs is a power of two, as the ue8m0 forms of the quantizers produce them; large problems then run with the scales
    inside the matrix instruction (``fg_block_fp8_gemm_pow2_scales``).  Scales of dtype ``float8_e8m0fnu`` carry
    that promise by construction.
    """
    logger.debug("GEMS W8A8_BLOCK_FP8_MATMUL")
    assert len(block_size) == 2
    block_n, block_k = block_size[0], block_size[1]

    assert A.shape[-1] == B.shape[-1]
    assert A.shape[:-1] == As.shape[:-1] and A.is_contiguous()
    assert _cdiv(A.shape[-1], block_k) == As.shape[-1]
    M = math.prod(A.shape[:-1])

    assert B.ndim == 2 and Bs.ndim == 2
    N, K = B.shape
    assert _cdiv(N, block_n) == Bs.shape[0]
    assert _cdiv(K, block_k) == Bs.shape[1]
    if A.dtype != torch.float8_e4m3fn or B.dtype != torch.float8_e4m3fn:
        raise NotImplementedError(f"w8a8_block_fp8_matmul: operands must be float8_e4m3fn, got {A.dtype}, {B.dtype}")
    if output_dtype not in _OUT_DTYPES:
        raise NotImplementedError(f"w8a8_block_fp8_matmul: unsupported output dtype {output_dtype}")
    e8m0 = getattr(torch, "float8_e8m0fnu", None)
    pow2 = scales_are_powers_of_two or (e8m0 is not None and As.dtype == e8m0 and Bs.dtype == e8m0)
    if As.dtype != torch.float32 or Bs.dtype != torch.float32:
        As, Bs = As.to(torch.float32), Bs.to(torch.float32)

    C_shape = A.shape[:-1] + (N,)
    C = A.new_empty(C_shape, dtype=output_dtype)
    if M == 0 or N == 0:
        return C
    if B.stride(1) != 1:
        B = B.contiguous()
    a2d = A if A.dim() == 2 else A.view(M, K)
    as2d = As if As.dim() == 2 else As.reshape(M, As.shape[-1])
    if (block_n, block_k) != (128, 128) and block_n % 128 == 0 and block_k % 128 == 0:
        as2d, Bs, block_n, block_k = _scales_at_128(as2d, Bs, N, K, block_n, block_k)
    # (any other block size goes to the library as it is: csrc/fp8_gemm_anyblock.hip serves it)
    _launch_block_gemm(a2d, B, as2d, Bs, C if C.dim() == 2 else C.view(M, N), block_n, block_k, pow2)
    return C


def _scales_at_128(as2d: torch.Tensor, bs: torch.Tensor, n: int, k: int, block_n: int, block_k: int):
    """Scale blocks that are whole multiples of 128 restated at the kernels' 128 x 128 granularity: every 128-wide
    piece of a larger block gets a copy of the block's scale, so each product is multiplied by the same fp32 value at
    the same place of the sum and the result is what a kernel with the larger blocks would give (the reference's
    kernel takes any ``block_size``: src/flag_gems/ops/w8a8_block_fp8_matmul.py:51-122)."""
    assert block_n > 0 and block_k > 0 and block_n % 128 == 0 and block_k % 128 == 0
    rn, rk = block_n // 128, block_k // 128
    kb, nb = _cdiv(k, 128), _cdiv(n, 128)
    if rk > 1:
        as2d = as2d.repeat_interleave(rk, dim=1)[:, :kb]
        bs = bs.repeat_interleave(rk, dim=1)[:, :kb]
    if rn > 1:
        bs = bs.repeat_interleave(rn, dim=0)[:nb]
    return as2d.contiguous(), bs.contiguous(), 128, 128


def fp8_matmul(
    a: torch.Tensor,
    a_s: torch.Tensor,
    b: torch.Tensor,
    b_s: torch.Tensor,
    scale_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Block-wise scaled FP8 matmul with 128-wide groups and bf16 output.

    a [..., K] e4m3fn contiguous, a_s [..., K/128], b [N, K] e4m3fn contiguous, b_s [N/128, K/128];
    scales given as float8_e8m0fnu are widened to fp32 first (and, being powers of two, may be applied inside the
    matrix instruction: ``fg_block_fp8_gemm_pow2_scales``).
    """
    logger.debug("GEMS FP8_MATMUL")
    assert b.ndim == 2
    assert a.is_contiguous() and b.is_contiguous()
    assert a_s.is_contiguous() and b_s.is_contiguous()
    K = a.size(-1)
    M = a.numel() // K
    N, K2 = b.shape
    assert K == K2
    pow2 = scale_dtype == torch.float8_e8m0fnu
    if pow2:
        a_s = a_s.to(torch.float32)
        b_s = b_s.to(torch.float32)
    C = torch.empty((*a.size()[:-1], N), device=a.device, dtype=torch.bfloat16)
    if M == 0 or N == 0:
        return C
    dev = a.device
    if dev.type != "cuda":
        _lib.require_gpu(a, "block fp8 gemm")
    # every operand is contiguous (asserted above), so the leading dimensions follow from the shapes: no views, no
    # stride queries (the reference's direct wrapper exists for the same reason: cpp/lib/fp8_matmul_direct.cpp:62-63)
    kb = a_s.numel() // M
    assert kb * M == a_s.numel(), "a_s must hold one row of scales per row of a"
    bs_cols = b_s.size(-1)
    _launch_raw(dev, a.data_ptr(), K, b.data_ptr(), K, a_s.data_ptr(), kb, 1, b_s.data_ptr(), bs_cols, 1,
                C.data_ptr(), N, _lib.FG_BF16, M, N, K, GROUP_SIZE, GROUP_SIZE, pow2)
    return C


def fp8_matmul_noop(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor) -> torch.Tensor:
    """Everything ``fp8_matmul`` does on the host and nothing on the device: the same checks, the same
    allocation, no launch.  The returned bf16 tensor ``[..., N]`` is uninitialised.  Timing it next to
    ``fp8_matmul`` separates the binding's overhead from the kernel's launch."""
    assert b.ndim == 2, "b must be 2D"
    assert a.is_contiguous() and b.is_contiguous(), "a and b must be contiguous"
    assert a_s.is_contiguous() and b_s.is_contiguous(), "a_s and b_s must be contiguous"
    K = a.size(-1)
    M = a.numel() // K if K else 0
    N = b.size(0)
    assert b.size(1) == K, "a and b must have the same K dimension"
    assert M == 0 or (a_s.numel() // M) * M == a_s.numel(), "a_s must hold one row of scales per row of a"
    return torch.empty((*a.size()[:-1], N), device=a.device, dtype=torch.bfloat16)
