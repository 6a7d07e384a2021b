"""Pins the GEMM functions of oracle/fp8_linear_oracle.py: two independent
algorithms against each other, a float64 triple loop on tiny shapes, and closed
forms a wrong index / dropped scale / transposed operand would break."""
import numpy as np
import pytest
import torch

from oracle import e4m3
from oracle import fp8_linear_oracle as O

FP8 = torch.float8_e4m3fn


def _inputs(m, n, k, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(m, k, generator=g).to(FP8)
    b = torch.randn(n, k, generator=g).to(FP8)
    kb, nb = (k + 127) // 128, (n + 127) // 128
    a_s = 0.01 * torch.rand(m, kb, generator=g) + 0.005
    b_s = 0.01 * torch.rand(nb, kb, generator=g) + 0.005
    return a, b, a_s, b_s


def _loop_f64(a, b, a_s, b_s):
    dec = e4m3.decode_table().astype(np.float64)
    an = dec[a.view(torch.uint8).numpy()]
    bn = dec[b.view(torch.uint8).numpy()]
    m, k = an.shape
    n = bn.shape[0]
    out = np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            acc = 0.0
            for kk in range(k):
                acc += an[i, kk] * bn[j, kk] * float(a_s[i, kk // 128]) * float(b_s[j // 128, kk // 128])
            out[i, j] = acc
    return out


@pytest.mark.parametrize("shape", [(3, 5, 128), (4, 130, 200), (2, 7, 300)])
def test_block_matmul_refs_vs_f64_loop(shape):
    m, n, k = shape
    a, b, a_s, b_s = _inputs(m, n, k, 11)
    want = _loop_f64(a, b, a_s, b_s)
    for fn in (O.block_fp8_matmul_dequant_ref, O.block_fp8_matmul_tiled_ref):
        got = fn(a, b, a_s, b_s, [128, 128], torch.float32).double().numpy()
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("shape", [(64, 512, 1024), (83, 260, 3884 // 4), (17, 2112, 512)])
def test_two_block_matmul_algorithms_agree(shape):
    m, n, k = shape
    a, b, a_s, b_s = _inputs(m, n, k, 12)
    x = O.block_fp8_matmul_dequant_ref(a, b, a_s, b_s, [128, 128], torch.float32)
    y = O.block_fp8_matmul_tiled_ref(a, b, a_s, b_s, [128, 128], torch.float32)
    z = O.block_fp8_matmul_dequant_ref(a, b, a_s, b_s, [128, 128], torch.float64, torch.float64)
    torch.testing.assert_close(x, y, rtol=1e-4, atol=1e-6)
    torch.testing.assert_close(x.double(), z, rtol=1e-4, atol=1e-6)


def test_unit_scales_reduce_to_plain_matmul():
    a, b, a_s, b_s = _inputs(16, 256, 384, 13)
    one_a, one_b = torch.ones_like(a_s), torch.ones_like(b_s)
    want = a.float() @ b.float().T  # exact: products of e4m3 values, small sums in fp32
    for fn in (O.block_fp8_matmul_dequant_ref, O.block_fp8_matmul_tiled_ref):
        got = fn(a, b, one_a, one_b, [128, 128], torch.float32)
        torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-4)


def test_one_hot_rows_pick_scaled_weight_entries():
    # A row with a single 1.0 at column c: C[m, n] = B[n, c] * As[m, c//128] * Bs[n//128, c//128]
    _, b, a_s, b_s = _inputs(4, 300, 512, 14)
    cols = [0, 127, 128, 511]
    a = torch.zeros(4, 512)
    for r, c in enumerate(cols):
        a[r, c] = 1.0
    a = a.to(FP8)
    for fn in (O.block_fp8_matmul_dequant_ref, O.block_fp8_matmul_tiled_ref):
        got = fn(a, b, a_s, b_s, [128, 128], torch.float32)
        for r, c in enumerate(cols):
            want = b[:, c].float() * a_s[r, c // 128] * b_s[:, c // 128].repeat_interleave(128)[:300]
            torch.testing.assert_close(got[r], want, rtol=1e-6, atol=0)


def test_power_of_two_scales_are_exact_and_k_block_specific():
    a, b, _, _ = _inputs(8, 128, 256, 15)
    a_s = torch.tensor([[2.0, 0.5]]).repeat(8, 1)
    b_s = torch.tensor([[0.25, 4.0]])
    af, bf = a.float(), b.float()
    want = (af[:, :128] @ bf[:, :128].T) * 0.5 + (af[:, 128:] @ bf[:, 128:].T) * 2.0
    for fn in (O.block_fp8_matmul_dequant_ref, O.block_fp8_matmul_tiled_ref):
        got = fn(a, b, a_s, b_s, [128, 128], torch.float32)
        torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-5)


def test_leading_dims_are_kept():
    a, b, a_s, b_s = _inputs(6, 130, 256, 16)
    got = O.block_fp8_matmul_tiled_ref(a.view(2, 3, 256), b, a_s.view(2, 3, 2), b_s, [128, 128], torch.bfloat16)
    assert got.shape == (2, 3, 130) and got.dtype == torch.bfloat16
    flat = O.block_fp8_matmul_tiled_ref(a, b, a_s, b_s, [128, 128], torch.bfloat16)
    assert torch.equal(got.view(6, 130), flat)


# ---------------------------------------------------------------- scaled_mm
def _smm_inputs(m, n, k, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(m, k, generator=g).to(FP8)
    b = torch.randn(k, n, generator=g).t().contiguous().t().to(FP8)  # column-major
    sa = torch.randn(m, 1, generator=g)
    sb = torch.randn(1, n, generator=g)
    bias = torch.randn(n, generator=g).bfloat16()
    return a, b, sa, sb, bias


def test_scaled_mm_refs_vs_f64_loop_and_each_other():
    a, b, sa, sb, bias = _smm_inputs(5, 9, 64, 21)
    dec = e4m3.decode_table().astype(np.float64)
    an = dec[a.view(torch.uint8).numpy()]
    bn = dec[b.view(torch.uint8).numpy()]
    want = np.zeros((5, 9))
    for i in range(5):
        for j in range(9):
            want[i, j] = sum(an[i, kk] * bn[kk, j] for kk in range(64)) * float(sa[i, 0]) * float(sb[0, j])
    got = O.scaled_mm_ref(a, b, sa, sb, torch.float32).double().numpy()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    got2 = O.scaled_mm_ref_postscale(a, b, sa, sb, None, torch.float32).double().numpy()
    np.testing.assert_allclose(got2, want, rtol=1e-6, atol=1e-6)
    # bias is added after the cast, in the output dtype
    with_bias = O.scaled_mm_ref(a, b, sa, sb, torch.bfloat16, bias)
    no_bias = O.scaled_mm_ref(a, b, sa, sb, torch.bfloat16)
    assert torch.equal(with_bias, no_bias + bias)


def test_scaled_mm_scalar_and_unit_scales():
    a, b, _, _, _ = _smm_inputs(7, 33, 128, 22)
    one = torch.ones(1)
    plain = a.float() @ b.float()
    torch.testing.assert_close(O.scaled_mm_ref(a, b, one, one, torch.float32), plain, rtol=0, atol=0)
    s = torch.tensor([0.5])
    torch.testing.assert_close(O.scaled_mm_ref(a, b, s, one, torch.float32), plain * 0.5, rtol=0, atol=0)
    # per-row scale really scales rows (a transposed broadcast would fail here)
    sa = torch.arange(1, 8).float().reshape(7, 1)
    torch.testing.assert_close(O.scaled_mm_ref(a, b, sa, one, torch.float32), plain * sa, rtol=1e-6, atol=1e-5)
    sb = torch.arange(1, 34).float().reshape(1, 33)
    torch.testing.assert_close(O.scaled_mm_ref(a, b, one, sb, torch.float32), plain * sb, rtol=1e-6, atol=1e-5)


def test_config1_pipeline_is_self_consistent():
    r = O.run_config1(0)
    assert r["xq"].shape == (64, 1024) and r["xs"].shape == (64, 8)
    assert r["wq"].shape == (512, 1024) and r["ws"].shape == (4, 8)
    assert r["c"].shape == (64, 512) and r["c"].dtype == torch.bfloat16
    # quantized linear approximates the bf16 linear: relative Frobenius error of fp8 (3 mantissa bits)
    want = r["x"].float() @ r["w"].float().T
    rel = (r["c"].float() - want).norm() / want.norm()
    assert rel < 0.05


# ---- grouped (mixture-of-experts) block GEMM


def _grouped_inputs(m, n, k, experts, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(m, k, generator=g).to(FP8)
    b = torch.randn(experts, n, k, generator=g).to(FP8)
    kb, nb = (k + 127) // 128, (n + 127) // 128
    a_s = 0.01 * torch.rand(m, kb, generator=g) + 0.005
    b_s = 0.01 * torch.rand(experts, nb, kb, generator=g) + 0.005
    return a, b, a_s, b_s


def test_grouped_ref_vs_f64_loop_on_ragged_segments():
    ends = torch.tensor([2, 2, 5, 6], dtype=torch.int32)  # segment 1 is empty, row 6 belongs to nobody
    a, b, a_s, b_s = _grouped_inputs(7, 130, 256, 4, 21)
    got = O.grouped_block_fp8_matmul_ref(a, b, a_s, b_s, ends, [128, 128]).double().numpy()
    begin = 0
    for e, end in enumerate(ends.tolist()):
        if end > begin:
            want = _loop_f64(a[begin:end], b[e], a_s[begin:end], b_s[e])
            np.testing.assert_allclose(got[begin:end], want, rtol=1e-5, atol=1e-7)
        begin = end
    assert not got[6].any()


def test_grouped_ref_vs_dequantised_matmul_per_segment():
    ends = torch.tensor([40, 41, 41, 100], dtype=torch.int32)
    a, b, a_s, b_s = _grouped_inputs(100, 260, 384, 4, 22)
    got = O.grouped_block_fp8_matmul_ref(a, b, a_s, b_s, ends, [128, 128])
    begin = 0
    for e, end in enumerate(ends.tolist()):
        if end > begin:
            want = O.block_fp8_matmul_dequant_ref(a[begin:end], b[e], a_s[begin:end], b_s[e], [128, 128])
            torch.testing.assert_close(got[begin:end], want, rtol=1e-4, atol=1e-6)
        begin = end


def test_grouped_ref_closed_forms():
    a, b, a_s, b_s = _grouped_inputs(50, 256, 256, 3, 23)
    plain = O.block_fp8_matmul_tiled_ref(a, b[1], a_s, b_s[1], [128, 128])
    # one group holding every row is the plain GEMM with that group's weights
    ends = torch.tensor([0, 50, 50], dtype=torch.int32)
    assert torch.equal(O.grouped_block_fp8_matmul_ref(a, b, a_s, b_s, ends, [128, 128]), plain)
    # the same weights in every group: the segment ends stop mattering
    same_b, same_s = b[1:2].expand(3, -1, -1), b_s[1:2].expand(3, -1, -1)
    for ends in ([7, 7, 50], [13, 30, 50], [50, 50, 50]):
        got = O.grouped_block_fp8_matmul_ref(a, same_b, a_s, same_s, torch.tensor(ends, dtype=torch.int32), [128, 128])
        torch.testing.assert_close(got, plain, rtol=1e-6, atol=1e-7)
    # swapping two groups' weights changes exactly those groups' rows
    ends = torch.tensor([10, 30, 50], dtype=torch.int32)
    base = O.grouped_block_fp8_matmul_ref(a, b, a_s, b_s, ends, [128, 128])
    swapped = O.grouped_block_fp8_matmul_ref(a, b[[2, 1, 0]], a_s, b_s[[2, 1, 0]], ends, [128, 128])
    assert torch.equal(base[10:30], swapped[10:30])
    assert not torch.equal(base[:10], swapped[:10]) and not torch.equal(base[30:], swapped[30:])


def test_moe_rows_are_cumulative_and_skewed():
    ends = O.make_moe_rows(4096, 8, 2, seed=0)
    assert ends.dtype == torch.int32 and ends.numel() == 8 and int(ends[-1]) == 8192
    counts = torch.diff(ends, prepend=torch.zeros(1, dtype=torch.int32))
    assert (counts >= 0).all() and counts.max() > 2 * counts.min()
    assert torch.equal(ends, O.make_moe_rows(4096, 8, 2, seed=0))


# ---- batched einsum


def test_einsum_ref_per_head_and_f64():
    xq, xs, yq, ys = O.make_fp8_einsum_inputs(5, 3, 256, 256, seed=31)
    got = O.fp8_block_einsum_ref(xq, xs, yq, ys, [128, 128])
    assert got.shape == (5, 3, 256)
    for head in range(3):
        want = O.block_fp8_matmul_tiled_ref(xq[:, head], yq[head], xs[:, head], ys[head], [128, 128])
        torch.testing.assert_close(got[:, head], want, rtol=1e-4, atol=1e-5)
    want = _loop_f64(xq[:2, 1].contiguous(), yq[1, :9].contiguous(), xs[:2, 1], ys[1])
    np.testing.assert_allclose(got[:2, 1, :9].double().numpy(), want, rtol=1e-5, atol=1e-6)
    # scales of this input maker are powers of two and every group's largest code is +-448 or the group is tiny
    assert torch.all(torch.frexp(xs)[0] == 0.5) and torch.all(torch.frexp(ys)[0] == 0.5)


def _moe_inputs(tokens, experts, hidden, inter, topk, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(tokens, hidden, generator=g).bfloat16()
    w1 = (torch.randn(experts, 2 * inter, hidden, generator=g) / hidden**0.5).to(FP8)
    w2 = (torch.randn(experts, hidden, inter, generator=g) / inter**0.5).to(FP8)
    s1 = torch.rand(experts, 2 * inter // 128, hidden // 128, generator=g) + 0.5
    s2 = torch.rand(experts, hidden // 128, inter // 128, generator=g) + 0.5
    gate = torch.randn(tokens, experts, generator=g)
    tw, ti = torch.topk(torch.softmax(gate, dim=-1), topk, dim=-1)
    tw = (tw / tw.sum(dim=-1, keepdim=True)).bfloat16()
    return x, w1, w2, s1, s2, tw, ti


def _dense_mlp_f64(x, w1, w2, s1, s2):
    """One expert's quantize -> GEMM -> SiLU-and-mul -> quantize -> GEMM through the *dequantised float64* GEMM
    oracle (an algorithm other than the tiled one the MoE restatement calls), rounded to bf16 where the layer
    rounds."""
    q, s = O.per_token_group_quant_fp8_div_ref(x.contiguous(), 128)
    h = O.block_fp8_matmul_dequant_ref(q, w1, s, s1, [128, 128], torch.bfloat16, torch.float64)
    q2, s2a = O.per_token_group_quant_fp8_div_ref(O.silu_and_mul_ref(h).contiguous(), 128)
    return O.block_fp8_matmul_dequant_ref(q2, w2, s2a, s2, [128, 128], torch.bfloat16, torch.float64)


def test_moe_ref_with_identical_experts_is_the_dense_layer():
    """Every expert holds the same weights and the routing weights of a token sum to one: whatever the routing, the
    layer is the dense MLP (a wrong slot -> token map, a dropped weight or a missed slot breaks this).  The GEMM
    results differ from the float64 route by a bf16 rounding here and there, which the second quantization can
    amplify to a few percent of a row's largest element."""
    x, w1, w2, s1, s2, tw, ti = _moe_inputs(12, 4, 256, 128, 2, seed=3)
    w1[:] = w1[0]; w2[:] = w2[0]; s1[:] = s1[0]; s2[:] = s2[0]
    got = O.block_fp8_moe_ref(x, w1, w2, s1, s2, tw, ti, [128, 128]).float()
    want = _dense_mlp_f64(x, w1[0], w2[0], s1[0], s2[0]).float()
    torch.testing.assert_close(got, want, rtol=3e-2, atol=3e-2 * float(want.abs().max()))


def test_moe_ref_top1_picks_the_routed_expert_and_the_map_zeroes_foreign_slots():
    x, w1, w2, s1, s2, _, _ = _moe_inputs(10, 3, 256, 128, 1, seed=5)
    ids = torch.tensor([0, 2, 1, 1, 0, 2, 2, 0, 1, 0]).view(-1, 1)
    ones = torch.ones(10, 1).bfloat16()
    got = O.block_fp8_moe_ref(x, w1, w2, s1, s2, ones, ids, [128, 128]).float()
    for e in range(3):
        rows = (ids[:, 0] == e).nonzero()[:, 0]
        want = _dense_mlp_f64(x[rows], w1[e], w2[e], s1[e], s2[e]).float()
        torch.testing.assert_close(got[rows], want, rtol=3e-2, atol=3e-2 * float(want.abs().max()))
    # half weights halve the result exactly (a power of two)
    half = O.block_fp8_moe_ref(x, w1, w2, s1, s2, 0.5 * ones, ids, [128, 128]).float()
    assert torch.equal(half, 0.5 * got)
    # global experts 0 and 2 live elsewhere; global 1 is local expert 0
    emap = torch.tensor([-1, 0, -1])
    local = O.block_fp8_moe_ref(x, w1[1:2], w2[1:2], s1[1:2], s2[1:2], ones, ids, [128, 128], expert_map=emap).float()
    mine = ids[:, 0] == 1
    assert torch.equal(local[mine], got[mine]) and float(local[~mine].abs().max()) == 0.0
    # a sample of tokens gives the rows of the full evaluation
    pick = torch.tensor([7, 2, 3])
    assert torch.equal(O.block_fp8_moe_ref(x, w1, w2, s1, s2, ones, ids, [128, 128], tokens=pick).float(), got[pick])
