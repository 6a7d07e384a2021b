"""GPU parity of the grouped (mixture-of-experts) block-scaled FP8 GEMM against the CPU oracle.

Tolerance: rtol 1e-2 / atol 1e-2 for the bf16 result against the per-group fp32 restatement of the
reference's MoE check (tests/test_fused_experts_impl.py:636-646); where a plain GEMM computes the same
tiles in the same order the results are compared bit for bit."""
import ctypes

import pytest
import torch

import flag_gems
from flaggems_amd import _lib
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn


def _inputs(M, N, K, E, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).bfloat16()
    xq, xs = O.act_quant_ref(x, 128)
    wq, ws = [], []
    for _ in range(E):
        q, s = O.per_block_cast_to_fp8_ref((0.02 * torch.randn(N, K, generator=g)).bfloat16())
        wq.append(q)
        ws.append(s)
    return xq, torch.stack(wq), xs, torch.stack(ws)


def _run(xq, wq, xs, ws, ends):
    return flag_gems.grouped_w8a8_block_fp8_matmul(
        xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), ends.to(DEV), [128, 128])


def _check(got, xq, wq, xs, ws, ends):
    want = O.grouped_block_fp8_matmul_ref(xq, wq, xs, ws, ends, [128, 128])
    rows = min(int(ends.max()), xq.shape[0])
    assert got.dtype == torch.bfloat16 and got.shape == want.shape
    torch.testing.assert_close(got.cpu().float()[:rows], want[:rows], rtol=1e-2, atol=1e-2)
    # at most one bf16 rounding plus fp32 accumulation noise
    err = (got.cpu().double()[:rows] - want.double()[:rows]).abs()
    assert float((err / (want[:rows].double().abs() / 128 + 2e-3)).max()) < 1.0


CASES = [
    # M, N, K, ends
    (1024, 640, 512, [300, 300, 301, 1000]),          # an empty group, a one-row group, rows nobody owns
    (128, 1024, 1024, None),                           # 64 tokens, top-2, 8 experts: every tile is mostly edge
    (2048, 2144, 1024, None),                          # N ends inside a scale block
    (3000, 6144, 256, [1000, 1900, 3000]),             # more tiles than compute units: blocks walk several
    (700, 384, 2048, [0, 0, 0, 0, 0, 0, 0, 700]),      # all rows in the last group
    (513, 256, 128, [256, 512, 513]),                  # segments that end on tile boundaries, one K-block
    # few rows per segment (64-row tiles), few tiles, deep K: the tiles are cut along K
    (128, 512, 4096, None),
    (96, 264, 2048, [0, 1, 1, 40, 40, 41, 90, 96]),    # N ends inside a tile; empty and one-row segments
    (300, 256, 3072, [0, 200, 200, 230, 299, 300, 300, 300]),  # a segment of several short tiles
    (16, 1024, 7168, None),                            # more segments than rows have tokens
    # 33 .. 128 rows per segment on average: 128-row tiles, also cut along K
    (512, 512, 4096, None),
    (1000, 2144, 1024, [90, 130, 400, 401, 401, 640, 880, 1000]),
]


@pytest.mark.parametrize("M,N,K,ends", CASES)
def test_grouped_gemm_matches_the_oracle(M, N, K, ends):
    ends = O.make_moe_rows(M // 2, 8, 2, seed=M) if ends is None else torch.tensor(ends, dtype=torch.int32)
    xq, wq, xs, ws = _inputs(M, N, K, ends.numel(), seed=N)
    got = _run(xq, wq, xs, ws, ends)
    _check(got, xq, wq, xs, ws, ends)
    # a second call gives the same bits (no order of arrival enters the sums)
    rows = int(ends[-1])  # rows nobody owns are left as torch.empty made them
    assert torch.equal(got[:rows], _run(xq, wq, xs, ws, ends)[:rows])


def test_grouped_gemm_equals_plain_gemm_where_the_tiles_coincide():
    """Segment ends on tile boundaries and the same weights in every group: the grouped kernel computes the tiles
    of the plain GEMM (256 of them, which the plain path gives whole to the persistent kernel), bit for bit."""
    M, N, K = 4096, 4096, 256
    xq, wq, xs, ws = _inputs(M, N, K, 1, seed=5)
    ends = torch.tensor([1024, 1024, 4096], dtype=torch.int32)
    got = _run(xq, wq.expand(3, -1, -1).contiguous(), xs, ws.expand(3, -1, -1).contiguous(), ends)
    plain = flag_gems.w8a8_block_fp8_matmul(xq.to(DEV), wq[0].to(DEV), xs.to(DEV), ws[0].to(DEV), [128, 128])
    assert torch.equal(got, plain)
    # ends inside tiles change which tile a row falls in, not its sums
    ends = torch.tensor([1000, 1001, 4096], dtype=torch.int32)
    got = _run(xq, wq.expand(3, -1, -1).contiguous(), xs, ws.expand(3, -1, -1).contiguous(), ends)
    assert torch.equal(got, plain)


@pytest.mark.parametrize("M,N,K,ends", [(16700, 1024, 4096, [5000, 5001, 16700]), (9000, 2048, 2048, [100, 4100, 4100, 9000])])
def test_last_round_of_256_row_tiles_is_cut_along_k(M, N, K, ends):
    """More 256-row tiles than compute units, a few of them left for a last round (268 = 256 + 12 and 296 = 256 + 40):
    those are cut into work items along K whose sums meet in the workspace.  Every row against the plain GEMM of its
    segment (another kernel instantiation; whole tiles give the same bits there, cut tiles sums in another order),
    sampled rows against the oracle, and the same bits on a second call."""
    g = torch.Generator().manual_seed(M)
    xq = torch.randn(M, K, generator=g).to(FP8)
    xs = torch.rand(M, K // 128, generator=g) * 0.02 + 0.005
    E = len(ends)
    wq = (0.5 * torch.randn(E, N, K, generator=g)).to(FP8)
    ws = torch.rand(E, N // 128, K // 128, generator=g) * 0.02 + 0.005
    ends_t = torch.tensor(ends, dtype=torch.int32)
    got = _run(xq, wq, xs, ws, ends_t)
    assert torch.equal(got, _run(xq, wq, xs, ws, ends_t))
    begin, same = 0, 0
    for e, end in enumerate(ends):
        if end > begin:
            plain = flag_gems.w8a8_block_fp8_matmul(xq[begin:end].to(DEV), wq[e].to(DEV), xs[begin:end].to(DEV), ws[e].to(DEV), [128, 128])
            torch.testing.assert_close(got[begin:end].float(), plain.float(), rtol=1e-2, atol=1e-2)
            same += int((got[begin:end] == plain).sum())
        begin = end
    assert same > 0.9 * M * N  # most tiles are whole and coincide bit for bit
    rows = torch.randperm(M, generator=g)[:96].sort().values
    seg = torch.bucketize(rows, ends_t.long(), right=True)
    for e in range(E):
        pick = rows[seg == e]
        if pick.numel():
            want = O.block_fp8_matmul_dequant_ref(xq[pick], wq[e], xs[pick], ws[e], [128, 128], torch.float32, torch.float64)
            torch.testing.assert_close(got[pick.to(DEV)].cpu().float(), want, rtol=1e-2, atol=1e-2)


def test_group_table_is_forced_into_range():
    """Ends that go backwards or past the rows are forced into [previous end, M]: no row is read or written
    outside the operands, and the result is that of the forced table."""
    M, N, K = 1000, 512, 256
    xq, wq, xs, ws = _inputs(M, N, K, 3, seed=8)
    got = _run(xq, wq, xs, ws, torch.tensor([500, 200, 5000], dtype=torch.int32))
    _check(got, xq, wq, xs, ws, torch.tensor([500, 500, 1000], dtype=torch.int32))


def test_scale_layouts_and_missing_workspace_through_the_c_abi():
    """Column-major activation scales are read in place; without a workspace row-major scales are read as they
    lie.  Both give the bits of the default call."""
    M, N, K, E = 1500, 768, 2048, 4
    ends = torch.tensor([100, 900, 900, 1500], dtype=torch.int32)
    xq, wq, xs, ws = _inputs(M, N, K, E, seed=9)
    base = _run(xq, wq, xs, ws, ends)
    _check(base, xq, wq, xs, ws, ends)
    xs_cm = xs.to(DEV).t().contiguous().t()
    assert xs_cm.stride() == (1, M)
    got = flag_gems.grouped_w8a8_block_fp8_matmul(xq.to(DEV), wq.to(DEV), xs_cm, ws.to(DEV), ends.to(DEV), [128, 128])
    assert torch.equal(got, base)
    a, b, a_s, b_s, e = xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), ends.to(DEV)
    c = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    st = _lib.load().fg_grouped_block_fp8_gemm(
        a.data_ptr(), K, b.data_ptr(), K, N * K, a_s.data_ptr(), a_s.stride(0), 1,
        b_s.data_ptr(), b_s.stride(1), 1, b_s.stride(0), e.data_ptr(), E, None, 1, M, 0, None,
        c.data_ptr(), N, _lib.DTYPE_CODE[torch.bfloat16], M, N, K, 128, 128,
        None, 0, _lib.current_stream_ptr(torch.device(DEV)))
    _lib.check(st, "fg_grouped_block_fp8_gemm")
    torch.cuda.synchronize()
    assert torch.equal(c, base)


def test_unsupported_requests_fail_loudly():
    xq, wq, xs, ws = _inputs(64, 256, 256, 2, seed=1)
    ends = torch.tensor([10, 64], dtype=torch.int32)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), ends.to(DEV))
    with pytest.raises(NotImplementedError):
        flag_gems.grouped_w8a8_block_fp8_matmul(*args, [128, 128], output_dtype=torch.float32)
    with pytest.raises(NotImplementedError):  # scale blocks other than 128 x 128
        flag_gems.grouped_w8a8_block_fp8_matmul(*args[:3], torch.ones(2, 4, 2, device=DEV), args[4], [64, 128])
    with pytest.raises(AssertionError):
        flag_gems.grouped_w8a8_block_fp8_matmul(*args[:4], ends.to(torch.int64).to(DEV), [128, 128])
    # K that is not a multiple of 128
    g = torch.Generator().manual_seed(2)
    a = torch.randn(64, 192, generator=g).to(FP8).to(DEV)
    b = torch.randn(2, 256, 192, generator=g).to(FP8).to(DEV)
    with pytest.raises(NotImplementedError):
        flag_gems.grouped_w8a8_block_fp8_matmul(a, b, torch.ones(64, 2, device=DEV), torch.ones(2, 2, 2, device=DEV),
                                                ends.to(DEV), [128, 128])


@pytest.mark.parametrize("T,N,K,top_k", [(64, 1024, 1024, 2), (700, 2144, 512, 2), (1500, 768, 2048, 1), (333, 640, 256, 4),
                                         (256, 1024, 1024, 2), (200, 512, 4096, 2)])
def test_rows_gathered_through_an_index(T, N, K, top_k):
    """row_index: the kernel reads row sorted_token_ids[m] // top_k of the token matrix for sorted row m, as the
    reference's MoE kernel does (src/flag_gems/fused/fused_moe.py:1111), instead of a copy of the activations in
    expert order.  The result must carry the bits of the call on the materialised copy, and match the oracle."""
    E = 8
    g = torch.Generator().manual_seed(T + N)
    xq, wq, xs, ws = _inputs(T, N, K, E, seed=T)
    # route every token to top_k experts; sorted_token_ids lists (token * top_k + slot) grouped by expert
    expert_of = torch.randint(0, E, (T * top_k,), generator=g)
    order = torch.argsort(expert_of, stable=True).to(torch.int32)          # sorted_token_ids
    ends = torch.cumsum(torch.bincount(expert_of, minlength=E), 0).to(torch.int32)
    src = (order // top_k).long()
    got = flag_gems.grouped_w8a8_block_fp8_matmul(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), ends.to(DEV), [128, 128],
                                                  row_index=order.to(DEV), index_divisor=top_k)
    assert got.shape == (T * top_k, N)
    a_sorted, s_sorted = xq.view(torch.uint8)[src].view(FP8), xs[src]
    _check(got, a_sorted, wq, s_sorted, ws, ends)
    materialised = _run(a_sorted, wq, s_sorted, ws, ends)
    assert torch.equal(got, materialised)
    # column-major scales of the token matrix are read in place, through the same index
    xs_cm = xs.to(DEV).t().contiguous().t()
    again = flag_gems.grouped_w8a8_block_fp8_matmul(xq.to(DEV), wq.to(DEV), xs_cm, ws.to(DEV), ends.to(DEV), [128, 128],
                                                    row_index=order.to(DEV), index_divisor=top_k)
    assert torch.equal(again, got)


def test_gather_index_is_forced_into_range():
    T, N, K, E = 100, 256, 256, 2
    xq, wq, xs, ws = _inputs(T, N, K, E, seed=3)
    idx = torch.tensor([5, -7, 99, 100, 10 ** 6, 0, 50, 51], dtype=torch.int32)
    ends = torch.tensor([3, 8], dtype=torch.int32)
    got = flag_gems.grouped_w8a8_block_fp8_matmul(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), ends.to(DEV), [128, 128],
                                                  row_index=idx.to(DEV))
    src = idx.long().clamp(0, T - 1)
    _check(got, xq.view(torch.uint8)[src].view(FP8), wq, xs[src], ws, ends)


def _aligned_layout(expert_of, E, block_m):
    """sorted_token_ids / cumulative ends in the layout of the reference's moe_align_block_size
    (src/flag_gems/fused/moe_align_block_size.py:404-517): slots grouped by expert, every expert padded to a multiple
    of block_m with the value numel."""
    numel = expert_of.numel()
    ids, ends, total = [], [], 0
    for e in range(E):
        mine = torch.nonzero(expert_of == e).flatten().to(torch.int32)
        pad = (-mine.numel()) % block_m
        ids += [mine, torch.full((pad,), numel, dtype=torch.int32)]
        total += mine.numel() + pad
        ends.append(total)
    return torch.cat(ids), torch.tensor(ends, dtype=torch.int32)


@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("T,N,K,top_k,block_m", [(64, 1024, 1024, 2, 16), (700, 2144, 512, 2, 64), (333, 640, 256, 4, 64),
                                                 (1500, 768, 2048, 1, 128), (256, 1024, 1024, 2, 32), (200, 512, 4096, 2, 16)])
def test_results_scattered_and_weighted_like_the_moe_kernel(T, N, K, top_k, block_m, weighted):
    """The whole GEMM of the reference's MoE kernel (src/flag_gems/fused/fused_moe.py:1084-1125, 1484-1509): rows read
    through sorted_token_ids // top_k, results written to row sorted_token_ids[m] of a [T * top_k, N] matrix, padding
    entries (value numel) skipped, and with MUL_ROUTED_WEIGHT the fp32 sums multiplied by the slot's routing weight
    before the cast.  Expected: the oracle's per-expert product of every slot's token, times the weight in fp32."""
    E = 8
    g = torch.Generator().manual_seed(T * 3 + N)
    xq, wq, xs, ws = _inputs(T, N, K, E, seed=T + 1)
    slots = T * top_k
    expert_of = torch.randint(0, E, (slots,), generator=g)
    expert_of[expert_of == 5] = 4                                   # an expert nobody is routed to
    sorted_ids, ends = _aligned_layout(expert_of, E, block_m)
    assert sorted_ids.numel() == int(ends[-1]) and sorted_ids.numel() % block_m == 0
    weights = torch.rand(slots, generator=g) + 0.25 if weighted else None
    got = flag_gems.grouped_w8a8_block_fp8_matmul(
        xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), ends.to(DEV), [128, 128], row_index=sorted_ids.to(DEV),
        index_divisor=top_k, scatter_rows=slots, row_weights=weights.to(DEV) if weighted else None)
    assert got.shape == (slots, N) and got.dtype == torch.bfloat16
    # oracle: slots in expert order without padding, then back to slot order
    order = torch.argsort(expert_of, stable=True)
    src = (order // top_k).long()
    plain_ends = torch.cumsum(torch.bincount(expert_of, minlength=E), 0).to(torch.int32)
    ref_sorted = O.grouped_block_fp8_matmul_ref(xq.view(torch.uint8)[src].view(FP8), wq, xs[src], ws, plain_ends, [128, 128])
    want = torch.empty(slots, N)
    want[order] = ref_sorted * (weights[order].unsqueeze(1) if weighted else 1.0)
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    err = (got.cpu().double() - want.double()).abs()
    assert float((err / (want.double().abs() / 128 + 2e-3)).max()) < 1.0
    # the same bits as the call that leaves the rows in sorted order, row by row (no weights: nothing but the row moves)
    if not weighted:
        in_order = flag_gems.grouped_w8a8_block_fp8_matmul(
            xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), ends.to(DEV), [128, 128], row_index=sorted_ids.to(DEV),
            index_divisor=top_k)
        real = (sorted_ids < slots).to(DEV)
        assert torch.equal(got[sorted_ids.to(DEV)[real].long()], in_order[real])
    again = flag_gems.grouped_w8a8_block_fp8_matmul(
        xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), ends.to(DEV), [128, 128], row_index=sorted_ids.to(DEV),
        index_divisor=top_k, scatter_rows=slots, row_weights=weights.to(DEV) if weighted else None)
    assert torch.equal(again, got)
    # index_divisor = 0: the rows are handed over in sorted order already and the index only addresses the result
    src_rows = (sorted_ids.clamp(0, slots - 1) // top_k).long()
    presorted = flag_gems.grouped_w8a8_block_fp8_matmul(
        xq.to(DEV)[src_rows.to(DEV)].contiguous(), wq.to(DEV), xs.to(DEV)[src_rows.to(DEV)].contiguous(), ws.to(DEV), ends.to(DEV),
        [128, 128], row_index=sorted_ids.to(DEV), index_divisor=0, scatter_rows=slots,
        row_weights=weights.to(DEV) if weighted else None)
    assert torch.equal(presorted, got)


def test_scatter_skips_padding_and_rows_out_of_range():
    """Entries outside [0, scatter_rows) store nothing: the rows they would have hit keep their contents."""
    T, N, K, E = 40, 256, 256, 2
    xq, wq, xs, ws = _inputs(T, N, K, E, seed=11)
    idx = torch.tensor([3, 40, -1, 7, 10 ** 6, 0, 39, 12], dtype=torch.int32)
    ends = torch.tensor([4, 8], dtype=torch.int32)
    lib = _lib.load()
    c = torch.full((T, N), 7.0, dtype=torch.bfloat16, device=DEV)
    a, b, a_s, b_s, e, ix = xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), ends.to(DEV), idx.to(DEV)
    st = lib.fg_grouped_block_fp8_gemm(
        a.data_ptr(), K, b.data_ptr(), K, N * K, a_s.data_ptr(), a_s.stride(0), 1,
        b_s.data_ptr(), b_s.stride(1), 1, b_s.stride(0), e.data_ptr(), E, ix.data_ptr(), 1, T, T, None,
        c.data_ptr(), N, _lib.DTYPE_CODE[torch.bfloat16], idx.numel(), N, K, 128, 128,
        None, 0, _lib.current_stream_ptr(torch.device(DEV)))
    _lib.check(st, "fg_grouped_block_fp8_gemm")
    torch.cuda.synchronize()
    written = [3, 7, 0, 39, 12]
    untouched = sorted(set(range(T)) - set(written))
    assert (c[untouched] == 7.0).all()
    src = idx.long().clamp(0, T - 1)
    ref = O.grouped_block_fp8_matmul_ref(xq.view(torch.uint8)[src].view(FP8), wq, xs[src], ws, ends, [128, 128])
    for m, row in enumerate(idx.tolist()):
        if 0 <= row < T:
            torch.testing.assert_close(c[row].cpu().float(), ref[m], rtol=1e-2, atol=1e-2)
