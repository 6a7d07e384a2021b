"""Grouped block-scaled FP8 GEMM for mixture-of-experts layers (host side).

The reference runs its block-fp8 experts through ``fused_moe_kernel``
(src/flag_gems/fused/fused_moe.py:1378-1450), which gathers token rows through
``sorted_token_ids``; its grouped GEMM operator ``aten::_scaled_grouped_mm``
(src/flag_gems/ops/scaled_grouped_mm.py:240-583) takes rows already sorted by group with a table
``offs`` of cumulative int32 row ends (:111-114, :275-287) but only row-wise scales.  This operator
joins the two: the 2-D x 3-D case of ``_scaled_grouped_mm`` (rows of ``A`` cut by ``offs``, one weight
matrix per group) with the 1 x 128 / 128 x 128 block scales of ``w8a8_block_fp8_matmul``.  ``offs``
stays on the device; the kernel reads it, so the call never synchronises.
"""
from __future__ import annotations

import logging
from typing import List, Optional

import torch

from . import _lib

logger = logging.getLogger("flag_gems." + __name__.split(".")[-1])


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def group_ends_from_expert_ids(expert_ids: torch.Tensor, block_m: int, num_experts: int) -> torch.Tensor:
    """The ``offs`` table of ``grouped_w8a8_block_fp8_matmul`` from the per-block expert table that the reference's
    ``moe_align_block_size`` returns WITHOUT an ``expert_map`` (one entry per ``block_m`` sorted rows, ascending
    expert ids, -1 only for the blocks past the padded end; src/flag_gems/fused/moe_align_block_size.py:404-517,
    consumed at src/flag_gems/fused/fused_moe.py:1105).  Expert e then ends after ``block_m`` times the number of
    blocks with an id in [0, e].  Stays on the device of ``expert_ids`` and does not synchronise.

    A table that went through ``expert_map`` (moe_align_block_size.py:817-818) can hold -1 in front of or between
    the local experts' blocks and local ids out of order; cumulative ends cannot express that.  Use
    ``local_rows_from_moe_align`` for such tables."""
    assert expert_ids.ndim == 1 and block_m >= 1 and num_experts >= 1
    ids = expert_ids.to(torch.int64)
    used = (ids >= 0) & (ids < num_experts)
    counts = torch.zeros(num_experts, dtype=torch.int64, device=expert_ids.device)
    counts.scatter_add_(0, ids.clamp(0, num_experts - 1), used.to(torch.int64))
    return (torch.cumsum(counts, 0) * block_m).to(torch.int32)


def local_rows_from_moe_align(sorted_token_ids: torch.Tensor, expert_ids: torch.Tensor, block_m: int, num_experts: int):
    """``(row_index, offs)`` for ``grouped_w8a8_block_fp8_matmul`` from the tables of the reference's
    ``moe_align_block_size`` after ``expert_map`` has been applied (src/flag_gems/fused/moe_align_block_size.py:
    771-819): ``expert_ids`` holds a LOCAL expert or -1 per block of ``block_m`` sorted rows, in any order.

    The blocks are reordered, ascending by local expert with the -1 blocks last (a stable sort of at most a few
    thousand block numbers on the device), and the rows of the -1 blocks are replaced by the padding value
    ``sorted_token_ids.numel()``: the GEMM never multiplies them and stores nothing for them.  The reference writes
    zeros for those rows (``write_zeros_to_output``, src/flag_gems/fused/fused_moe.py:804-820, 1114); pass
    ``zero_unwritten_rows=True`` to the GEMM for the same result.  No synchronisation."""
    assert sorted_token_ids.ndim == 1 and expert_ids.ndim == 1 and block_m >= 1 and num_experts >= 1
    nb = expert_ids.numel()
    n_sorted = sorted_token_ids.numel()
    # (the reference allocates numel + num_experts * (block_m - 1) sorted entries and one expert id per started block:
    # the last block may be short unless pad_sorted_ids was set; its missing entries count as padding)
    assert (nb - 1) * block_m < n_sorted <= nb * block_m, "one expert id per (started) block of block_m sorted rows"
    if n_sorted < nb * block_m:
        sorted_token_ids = torch.cat([sorted_token_ids, sorted_token_ids.new_full((nb * block_m - n_sorted,), n_sorted)])
    ids = expert_ids.to(torch.int64)
    local = (ids >= 0) & (ids < num_experts)
    key = torch.where(local, ids, torch.full_like(ids, num_experts))
    order = torch.argsort(key, stable=True)
    rows = sorted_token_ids.view(nb, block_m).to(torch.int32)
    pad = torch.full_like(rows, n_sorted)
    rows = torch.where(local[:, None], rows, pad)[order].reshape(-1).contiguous()
    counts = torch.zeros(num_experts + 1, dtype=torch.int64, device=expert_ids.device)
    counts.scatter_add_(0, key, torch.ones_like(key))
    offs = (torch.cumsum(counts[:num_experts], 0) * block_m).to(torch.int32)
    return rows, offs


def grouped_w8a8_block_fp8_matmul(
    A: torch.Tensor,
    B: torch.Tensor,
    As: torch.Tensor,
    Bs: torch.Tensor,
    offs: torch.Tensor,
    block_size: List[int],
    output_dtype: torch.dtype = torch.bfloat16,
    row_index: Optional[torch.Tensor] = None,
    index_divisor: int = 1,
    scatter_rows: Optional[int] = None,
    row_weights: Optional[torch.Tensor] = None,
    zero_unwritten_rows: bool = False,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """C[offs[e-1]:offs[e]] = block_fp8_matmul(A[offs[e-1]:offs[e]], B[e]) for every group e.

    A [M, K] contiguous e4m3fn (rows sorted by group), As [M, K/block_k] fp32, B [E, N, K] e4m3fn,
    Bs [E, ceil(N/block_n), K/block_k] fp32, offs [E] int32 cumulative row ends on A's device.
    Returns bf16 [M, N]; rows at or past offs[-1] are left unwritten (as ``torch.empty`` made them).

    With ``row_index`` (int32 [M] on A's device) the kernel gathers its rows itself: sorted row m is row
    ``row_index[m] // index_divisor`` of ``A [T, K]`` and ``As [T, K/block_k]``, the way the reference's MoE kernel
    reads its tokens (``sorted_token_ids // top_k``, src/flag_gems/fused/fused_moe.py:1111); the result still has
    M = ``row_index.numel()`` rows in sorted order.

    ``index_divisor=0`` (with ``scatter_rows``): A and As are in sorted order themselves and ``row_index`` only says
    where the results go -- the second GEMM of an expert layer whose intermediate rows stayed in expert order.

    With ``scatter_rows`` = R as well, the result has R rows and sorted row m is written to row ``row_index[m]``;
    entries outside ``[0, R)`` are padding (the reference pads ``sorted_token_ids`` with ``numel``,
    src/flag_gems/fused/moe_align_block_size.py:404-517) and store nothing, rows no entry names keep what
    ``torch.empty`` gave them.  ``row_weights`` (fp32 [R]) multiplies the fp32 sums of sorted row m by
    ``row_weights[row_index[m]]`` before the cast.  Both follow the epilogue of the reference's MoE kernel
    (src/flag_gems/fused/fused_moe.py:1484-1509: ``offs_token``, ``token_mask``, ``MUL_ROUTED_WEIGHT``).

    ``zero_unwritten_rows``: the result starts as zeros instead of ``torch.empty``, so rows that no group covers (the
    slots of experts that live on another device) read as zeros, which is what the reference's kernel stores for
    them (src/flag_gems/fused/fused_moe.py:1114).  ``out``: write into this ``[rows, N]`` tensor instead of a new one.
    """
    logger.debug("GEMS GROUPED_W8A8_BLOCK_FP8_MATMUL")
    assert len(block_size) == 2
    block_n, block_k = block_size[0], block_size[1]
    assert A.ndim == 2 and B.ndim == 3 and As.ndim == 2 and Bs.ndim == 3
    assert A.is_contiguous()
    T, K = A.shape  # rows of A: the sorted rows themselves, or the tokens they are gathered from
    M = T
    if row_index is not None:
        assert row_index.ndim == 1 and row_index.dtype == torch.int32 and row_index.is_contiguous()
        assert row_index.device == A.device and index_divisor >= 0
        M = row_index.numel()
        if index_divisor == 0:  # rows already in sorted order: the index only addresses the scattered result
            assert scatter_rows is not None and T == M, "index_divisor=0 needs scatter_rows and A in sorted order"

    c_rows = 0
    if scatter_rows is not None:
        assert row_index is not None, "scattered results are addressed through row_index"
        assert scatter_rows >= 1
        c_rows = int(scatter_rows)
    if row_weights is not None:
        assert c_rows > 0, "row_weights are indexed like the scattered result"
        assert row_weights.shape == (c_rows,) and row_weights.dtype == torch.float32 and row_weights.is_contiguous()
        assert row_weights.device == A.device
    E, N, K2 = B.shape
    assert K == K2
    assert As.shape[0] == T and As.shape[1] == _cdiv(K, block_k)
    assert Bs.shape == (E, _cdiv(N, block_n), _cdiv(K, block_k))
    assert offs.ndim == 1 and offs.numel() == E and offs.dtype == torch.int32
    assert offs.device == A.device and offs.is_contiguous()
    if A.dtype != torch.float8_e4m3fn or B.dtype != torch.float8_e4m3fn:
        raise NotImplementedError(f"grouped_w8a8_block_fp8_matmul: operands must be float8_e4m3fn, got {A.dtype}, {B.dtype}")
    if output_dtype not in (torch.bfloat16, torch.float16):
        raise NotImplementedError(f"grouped_w8a8_block_fp8_matmul: output dtype {output_dtype} (bfloat16 or float16)")
    if As.dtype != torch.float32 or Bs.dtype != torch.float32:
        As, Bs = As.to(torch.float32), Bs.to(torch.float32)
    if B.stride(2) != 1:
        B = B.contiguous()

    if out is not None:  # the caller's buffer: [rows, N] with unit stride along N
        assert out.shape == (c_rows if c_rows else M, N) and out.dtype == output_dtype and out.device == A.device
        assert out.stride(1) == 1
        C = out.zero_() if zero_unwritten_rows else out
    else:
        C = (A.new_zeros if zero_unwritten_rows else A.new_empty)((c_rows if c_rows else M, N), dtype=output_dtype)
    if M == 0 or N == 0:
        return C
    _lib.require_gpu(A, "grouped block fp8 gemm")
    lib = _lib.load()
    dev = A.device
    with _lib.device_guard(dev):
        ws_bytes = _lib.cached_workspace_bytes("fg_grouped_block_fp8_gemm_workspace_bytes", max(M, T), N, K)
        ws = _lib.workspace(dev, ws_bytes) if ws_bytes else None
        status = lib.fg_grouped_block_fp8_gemm(
            A.data_ptr(), A.stride(0) if T > 1 else max(K, A.stride(0)),
            B.data_ptr(), B.stride(1) if N > 1 else max(K, B.stride(1)), B.stride(0) if E > 1 else N * K,
            As.data_ptr(), As.stride(0), As.stride(1),
            Bs.data_ptr(), Bs.stride(1), Bs.stride(2), Bs.stride(0),
            offs.data_ptr(), E,
            row_index.data_ptr() if row_index is not None else None, index_divisor, T,
            c_rows, row_weights.data_ptr() if row_weights is not None else None,
            C.data_ptr(), C.stride(0), _lib.DTYPE_CODE[C.dtype],
            M, N, K, block_n, block_k,
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            _lib.current_stream_ptr(dev),
        )
    _lib.check(status, "fg_grouped_block_fp8_gemm")
    return C
