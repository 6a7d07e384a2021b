"""CPU-only checks: the shared library loads and exports every symbol the header declares, the
Python host mirrors the reference's argument checking before any launch, and importing the
package needs neither a GPU nor the library."""
import ctypes
import os
import re

import pytest
import torch

import flag_gems
import flaggems_amd
from flaggems_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = "".join(open(os.path.join(ROOT, "include", name)).read() for name in sorted(os.listdir(os.path.join(ROOT, "include")))
                   if name.endswith(".h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fg_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_all_bound_and_exported():
    declared = _declared_symbols()
    assert declared == sorted(_lib.SIGNATURES), "ctypes table and header disagree"
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("shared library not built on this host")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert _lib.load().fg_version() >= 100
    assert _lib.load().fg_last_error_string() is not None


def test_c_abi_argument_validation_needs_no_gpu():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("shared library not built on this host")
    lib = _lib.load()
    # cols not divisible by the group size -> FG_ERR_INVALID_ARG before any launch
    rc = lib.fg_group_quant_fp8(1, _lib.FG_BF16, 4, 100, 100, 1, _lib.FG_FP8_E4M3FN, 100, 1, 1, 1,
                                128, 1e-4, -448.0, 448.0, 1.0 / 448.0, 0, 0, 0, None)
    assert rc == _lib.FG_ERR_INVALID_ARG
    assert b"divisible" in lib.fg_last_error_string()
    # a scale block of no size is refused before any launch (every positive size is served)
    rc = lib.fg_block_fp8_gemm(1, 128, 1, 128, 1, 1, 1, 1, 1, 1, 1, 128, _lib.FG_BF16, 4, 4, 128, 0, 64, None, 0, None)
    assert rc == _lib.FG_ERR_INVALID_ARG
    assert b"scale block" in lib.fg_last_error_string()
    rc = lib.fg_block_fp8_gemm(None, 128, None, 128, None, 1, 1, None, 1, 1, None, 128, _lib.FG_BF16, 4, 4, 128, 128, 128, None, 0, None)
    assert rc == _lib.FG_ERR_INVALID_ARG
    # empty problems are accepted without touching the device
    assert lib.fg_group_quant_fp8(None, _lib.FG_BF16, 0, 128, 128, None, _lib.FG_FP8_E4M3FN, 128, None, 1, 1,
                                  128, 1e-4, -448.0, 448.0, 1.0 / 448.0, 0, 0, 0, None) == 0
    assert lib.fg_scaled_fp8_gemm(None, 0, None, 0, None, 0, None, 0, None, 0, None, 0, _lib.FG_BF16, 0, 8, 8, None, 0, None) == 0


def test_public_surface_matches_the_reference_names():
    for name in ["act_quant_triton", "per_token_group_quant_fp8", "SUPPORTED_FP8_DTYPE", "w8a8_block_fp8_matmul",
                 "fp8_matmul", "cutlass_scaled_mm", "scaled_mm", "scaled_mm_out", "enable", "only_enable", "use_gems",
                 "all_registered_ops", "all_registered_keys", "patch_empty_vllm"]:
        assert hasattr(flag_gems, name), name
    assert flag_gems.SUPPORTED_FP8_DTYPE == torch.float8_e4m3fn
    assert flag_gems.act_quant_triton is flaggems_amd.act_quant_triton


def test_no_cpu_fallback():
    x = torch.zeros(2, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        flag_gems.act_quant_triton(x)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        flag_gems.per_token_group_quant_fp8(x, 128)
    a = torch.zeros(2, 128, dtype=torch.float8_e4m3fn)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        flag_gems.w8a8_block_fp8_matmul(a, a, torch.ones(2, 1), torch.ones(1, 1), [128, 128])


def test_assertions_fire_before_any_launch():
    x = torch.zeros(4, 100, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="divisible by block_size"):
        flag_gems.act_quant_triton(x, 128)
    with pytest.raises(AssertionError, match="contiguous"):
        flag_gems.act_quant_triton(torch.zeros(128, 4, dtype=torch.bfloat16).t(), 128)
    with pytest.raises(AssertionError, match="must be divisible"):
        flag_gems.per_token_group_quant_fp8(x, 128)
    with pytest.raises(AssertionError, match="groups must be contiguous"):
        flag_gems.per_token_group_quant_fp8(torch.zeros(128, 4, dtype=torch.bfloat16).t(), 128)
    a = torch.zeros(4, 256, dtype=torch.float8_e4m3fn)
    with pytest.raises(AssertionError):
        flag_gems.w8a8_block_fp8_matmul(a, a[:, :128], torch.ones(4, 2), torch.ones(1, 1), [128, 128])
    with pytest.raises(AssertionError):
        flag_gems.w8a8_block_fp8_matmul(a, a, torch.ones(4, 3), torch.ones(1, 2), [128, 128])
    c = torch.zeros(4, 4, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="column-major"):
        flag_gems.cutlass_scaled_mm(c, a, torch.zeros(256, 4, dtype=torch.float8_e4m3fn), torch.ones(1), torch.ones(1))
    with pytest.raises(AssertionError, match="2D"):
        flag_gems.cutlass_scaled_mm(c, a[0], a, torch.ones(1), torch.ones(1))
    with pytest.raises(RuntimeError, match="cannot be multiplied"):
        flag_gems.scaled_mm(a, a, torch.ones(1), torch.ones(1))
    with pytest.raises(RuntimeError, match="scale_a must be"):
        flag_gems.scaled_mm(a, a.t(), torch.ones(3), torch.ones(1))


def test_registration_roundtrip_on_cpu_host():
    with flag_gems.use_gems():
        assert flag_gems.all_registered_keys() == ["_scaled_mm", "_scaled_mm.out"]
        assert flag_gems.all_registered_ops() == ["scaled_mm", "scaled_mm_out"]
    assert flag_gems.all_registered_keys() == []
    with flag_gems.use_gems(include=["scaled_mm"]):
        assert flag_gems.all_registered_keys() == ["_scaled_mm"]
    with flag_gems.use_gems(exclude=["scaled_mm_out"]):
        assert flag_gems.all_registered_keys() == ["_scaled_mm"]
    flag_gems.patch_empty_vllm()
    flag_gems.patch_empty_vllm()
    assert hasattr(torch.ops._C, "cutlass_scaled_mm") and hasattr(torch.ops._C, "per_token_group_fp8_quant")


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "flaggems_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, os.path.join(dirpath, f)


def test_widened_entry_points_validate_and_refuse_the_cpu():
    """The operators added around the hot path (grouped and batched GEMM, weight quantizer, fused activation, int8):
    same rules as the rest -- host checks first, no CPU implementation, C-ABI validation before any launch."""
    for name in ["grouped_w8a8_block_fp8_matmul", "w8a8_block_fp8_bmm", "fp8_einsum", "per_block_cast_to_fp8",
                 "per_token_cast_to_fp8", "silu_and_mul_packed", "silu_and_mul_per_token_group_quant_fp8"]:
        assert hasattr(flag_gems, name), name
    a = torch.zeros(4, 256, dtype=torch.float8_e4m3fn)
    b = torch.zeros(2, 128, 256, dtype=torch.float8_e4m3fn)
    ends = torch.tensor([1, 4], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        flag_gems.grouped_w8a8_block_fp8_matmul(a, b, torch.ones(4, 2), torch.ones(2, 1, 2), ends, [128, 128])
    with pytest.raises(AssertionError):  # the group table must be int32
        flag_gems.grouped_w8a8_block_fp8_matmul(a, b, torch.ones(4, 2), torch.ones(2, 1, 2), ends.long(), [128, 128])
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        flag_gems.fp8_einsum("bhr,hdr->bhd", torch.zeros(3, 2, 256, dtype=torch.float8_e4m3fn), torch.ones(3, 2, 2),
                             b, torch.ones(2, 1, 2))
    with pytest.raises(AssertionError, match="only supports"):
        flag_gems.fp8_einsum("bhr,hrd->bhd", torch.zeros(3, 2, 256, dtype=torch.float8_e4m3fn), torch.ones(3, 2, 2),
                             b, torch.ones(2, 1, 2))
    x = torch.zeros(4, 512, dtype=torch.bfloat16)
    for fn in (lambda: flag_gems.per_block_cast_to_fp8(x), lambda: flag_gems.per_token_cast_to_fp8(x),
               lambda: flag_gems.silu_and_mul_packed(x), lambda: flag_gems.silu_and_mul_per_token_group_quant_fp8(x, 128)):
        with pytest.raises(RuntimeError, match="no CPU implementation"):
            fn()
    with pytest.raises(AssertionError, match="divisible"):
        flag_gems.silu_and_mul_per_token_group_quant_fp8(x, 96)
    ai = torch.zeros(4, 256, dtype=torch.int8)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        flag_gems.cutlass_scaled_mm(torch.zeros(4, 16, dtype=torch.bfloat16), ai, torch.zeros(16, 256, dtype=torch.int8).t(),
                                    torch.ones(1), torch.ones(1))
    if not os.path.exists(_lib.LIB_PATH):
        return
    lib = _lib.load()
    # grouped GEMM: K that is not a multiple of 128, a non-bf16 result, a missing table
    args = lambda k, dt, tab: (1, k, 1, k, 128 * k, 1, 2, 1, 1, 2, 1, 2, tab, 2, None, 1, 4, 0, None, 1, 128, dt, 4, 128, k, 128, 128, None, 0, None)
    assert lib.fg_grouped_block_fp8_gemm(*args(192, _lib.FG_BF16, 1)) == _lib.FG_ERR_UNSUPPORTED
    assert lib.fg_grouped_block_fp8_gemm(*args(256, _lib.FG_F32, 1)) == _lib.FG_ERR_UNSUPPORTED
    assert lib.fg_grouped_block_fp8_gemm(*args(256, _lib.FG_BF16, None)) == _lib.FG_ERR_INVALID_ARG
    # scattered results need the index they are addressed through; row weights need scattered results
    bad = list(args(256, _lib.FG_BF16, 1))
    bad[17] = 8
    assert lib.fg_grouped_block_fp8_gemm(*bad) == _lib.FG_ERR_INVALID_ARG
    bad[17], bad[18] = 0, 1
    assert lib.fg_grouped_block_fp8_gemm(*bad) == _lib.FG_ERR_INVALID_ARG
    # block quantizer: only 128 x 128 blocks; empty input is accepted
    q = lambda rows, blk: lib.fg_block_quant_fp8(1, _lib.FG_BF16, rows, 256, 256, 1, _lib.FG_FP8_E4M3FN, 256, 1, 2, 1,
                                                 blk, blk, 1e-4, -448.0, 448.0, 1.0 / 448.0, 1, 0, 0, None)
    assert q(4, 64) == _lib.FG_ERR_UNSUPPORTED and q(0, 128) == 0
    # fused activation: the up half must lie inside the row
    rc = lib.fg_silu_mul_group_quant_fp8(1, _lib.FG_BF16, 4, 256, 300, 256, 1, _lib.FG_FP8_E4M3FN, 256, 1, 2, 1,
                                         128, 1e-10, -448.0, 448.0, 1.0 / 448.0, 0, 1, 0, None)
    assert rc == _lib.FG_ERR_INVALID_ARG
    assert lib.fg_batched_block_fp8_gemm(None, 0, 0, None, 0, 0, None, 0, 0, 0, None, 0, 0, 0, None, 0, 0, _lib.FG_BF16,
                                         -1, 4, 4, 128, 128, 128, None, 0, None) == _lib.FG_ERR_INVALID_ARG


def test_batched_workspace_query_is_host_only_and_never_below_the_single_problem():
    """fg_batched_block_fp8_gemm_workspace_bytes needs no GPU; it is at least the single-problem figure (with less the
    batched call takes a slower kernel, it never fails) and does not shrink when the batch grows past one entry's plan."""
    lib = _lib.load()
    for (M, N, K) in [(1, 1024, 4096), (8, 1024, 7168), (32, 128, 512), (64, 1024, 7168), (128, 1024, 4096), (4096, 1024, 4096)]:
        single = lib.fg_block_fp8_gemm_workspace_bytes(M, N, K)
        assert lib.fg_batched_block_fp8_gemm_workspace_bytes(1, M, N, K) == single
        for batch in (2, 8, 16, 128):
            assert lib.fg_batched_block_fp8_gemm_workspace_bytes(batch, M, N, K) >= single
    assert lib.fg_batched_block_fp8_gemm_workspace_bytes(16, 64, 1024, 7168) > lib.fg_block_fp8_gemm_workspace_bytes(64, 1024, 7168)


def test_group_ends_from_the_per_block_expert_table():
    """expert_ids as the reference's moe_align_block_size lays it out (one entry per block of sorted rows, experts
    ascending, -1 past the padded end) -> cumulative row ends per expert."""
    ids = torch.tensor([0, 0, 2, 3, 3, 3, -1, -1], dtype=torch.int32)
    ends = flag_gems.group_ends_from_expert_ids(ids, 64, 5)
    assert ends.dtype == torch.int32 and ends.tolist() == [128, 128, 192, 384, 384]
    assert flag_gems.group_ends_from_expert_ids(torch.tensor([-1], dtype=torch.int32), 16, 2).tolist() == [0, 0]


def test_local_rows_from_the_aligners_tables_on_the_host():
    """The reorder of an aligner table (pure torch, so it runs here): foreign (-1) blocks in front of and between
    the local experts' blocks, local ids out of order, and the reference's unpadded table length
    (numel + num_experts * (block_m - 1) entries, the last block short)."""
    block_m = 4
    expert_ids = torch.tensor([-1, 1, 0, -1, 1], dtype=torch.int32)
    sorted_ids = torch.arange(100, 100 + 18, dtype=torch.int32)  # 18 entries: the fifth block has 2 of its 4
    rows, offs = flag_gems.local_rows_from_moe_align(sorted_ids, expert_ids, block_m, 2)
    pad = 18
    assert offs.tolist() == [4, 12]                      # one block of expert 0, two of expert 1
    assert rows.tolist() == ([108, 109, 110, 111]        # expert 0: block 2
                             + [104, 105, 106, 107]      # expert 1: blocks 1 and 4, in table order
                             + [116, 117, pad, pad]
                             + [pad] * 8)                # the two foreign blocks, turned into padding
    with pytest.raises(AssertionError):
        flag_gems.local_rows_from_moe_align(sorted_ids[:16], expert_ids, block_m, 2)  # a whole block without entries


def test_record_once_lists_every_call_site_once(tmp_path):
    """enable(record=True, once=True): the record file names each operator call site once, however often it runs
    (the reference's LogOncePerLocationFilter, src/flag_gems/logging_utils.py:34-45); once=False lists every call."""
    import logging

    from flaggems_amd import registration

    child = logging.getLogger("flag_gems.some_operator")
    for once, want in ((True, 2), (False, 4)):
        path = tmp_path / f"ops_{once}.log"
        registration._setup_logging(True, once, str(path))
        try:
            for _ in range(3):
                child.debug("GEMS SOME_OPERATOR")   # one call site, three calls
            child.debug("GEMS SOME_OPERATOR")       # another call site
        finally:
            registration._teardown_logging()
        lines = path.read_text().splitlines()
        assert len(lines) == want, lines
        assert lines[0] == "[DEBUG] flag_gems.some_operator.test_record_once_lists_every_call_site_once: GEMS SOME_OPERATOR"
    assert not [h for h in logging.getLogger("flag_gems").handlers if h.get_name() == "flag_gems_record"]


def test_fastcall_module_marshals_the_decode_critical_calls():
    """csrc/fastcall.c: the CPython module through which the hosts of the block GEMM, the group quantizer and the
    scaled GEMM call the C ABI (a ctypes call spends 2-3 us on converting their 20-odd arguments).  On a host without
    a GPU only calls that launch nothing can run: empty problems return FG_OK, a wrong argument count raises."""
    import pytest

    from flaggems_amd import _lib

    f = _lib.fast()
    assert f.block_fp8_gemm(_lib.address("fg_block_fp8_gemm"), None, 0, None, 0, None, 0, 0, None, 0, 0, None, 0, _lib.FG_BF16,
                            0, 8, 128, 128, 128, None, 0, None) == _lib.FG_OK
    # a negative size comes back as the library's status, with its message behind fg_last_error_string
    assert f.block_fp8_gemm(_lib.address("fg_block_fp8_gemm"), None, 0, None, 0, None, 0, 0, None, 0, 0, None, 0, _lib.FG_BF16,
                            -1, 8, 128, 128, 128, None, 0, None) == _lib.FG_ERR_INVALID_ARG
    assert b"negative" in _lib.load().fg_last_error_string()
    assert f.group_quant_fp8(_lib.address("fg_group_quant_fp8"), None, _lib.FG_BF16, 0, 0, 0, None, _lib.FG_FP8_E4M3FN, 0, None, 0, 1,
                             128, 1e-10, -448.0, 448.0, 1.0 / 448.0, 0, 1, 0, None) == _lib.FG_OK
    assert f.scaled_gemm(_lib.address("fg_scaled_fp8_gemm"), None, 0, None, 0, None, 0, None, 0, None, 0, None, 0, _lib.FG_BF16,
                         0, 8, 128, None, 0, None) == _lib.FG_OK
    with pytest.raises(TypeError):
        f.block_fp8_gemm(_lib.address("fg_block_fp8_gemm"), 1, 2, 3)
    with pytest.raises(TypeError):
        f.scaled_gemm(_lib.address("fg_scaled_fp8_gemm"), "not a pointer", 0, None, 0, None, 0, None, 0, None, 0, None, 0, 0, 0, 8, 128, None, 0, None)
