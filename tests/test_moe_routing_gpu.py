"""GPU parity of the routing operators topk_softmax and grouped_topk against the CPU oracle's restatement of the
reference's kernels.  Indices must be equal; weights are floating point (an exponential, sums in another order): the bar
is the reference's own, atol 1e-5 for topk_softmax (tests/test_topk_softmax.py:101-103) and atol / rtol by type for
grouped_topk (tests/test_grouped_topk.py:59-72: 5e-3 / 1e-3 for 16-bit scores, 1e-5 .. 5e-4 for fp32).  Where two
probabilities of the oracle are closer than rounding can tell apart, either order is accepted."""
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _assert_same_choice(got_idx, want_idx, want_vals, what, slack=4e-7):
    """Equal indices, except where the oracle's own values at the two positions are within `slack` of each other."""
    got_idx, want_idx = got_idx.cpu().long(), want_idx.long()
    if torch.equal(got_idx, want_idx):
        return
    rows = (got_idx != want_idx).any(dim=1).nonzero().flatten()
    for r in rows.tolist():
        a, b = got_idx[r], want_idx[r]
        for pos in (a != b).nonzero().flatten().tolist():
            # the expert chosen here must be one the oracle ranks at a value indistinguishable from this position's
            where = (b == a[pos]).nonzero().flatten()
            assert where.numel() == 1, f"{what}: row {r} picks expert {a[pos].item()} that the oracle does not"
            gap = (want_vals[r, where[0]] - want_vals[r, pos]).abs().item()
            assert gap <= slack * max(1.0, want_vals[r, pos].abs().item()), f"{what}: row {r} position {pos}: gap {gap:.3e}"


@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64, torch.uint32])
@pytest.mark.parametrize("num_tokens, num_experts, topk", [(1, 4, 2), (4, 8, 2), (8, 16, 4), (32, 64, 8), (128, 128, 16),
                                                           (500, 255, 30), (512, 256, 32), (1024, 512, 32), (7, 1000, 5)])
@pytest.mark.parametrize("input_dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("renormalize", [False, True])
def test_topk_softmax(num_tokens, num_experts, topk, input_dtype, index_dtype, renormalize):
    g = torch.Generator().manual_seed(42)
    gating = torch.randn(num_tokens, num_experts, generator=g).to(input_dtype)
    w = torch.empty(num_tokens, topk, device=DEV, dtype=torch.float32)
    idx = torch.empty(num_tokens, topk, device=DEV, dtype=index_dtype)
    src = torch.empty(num_tokens, topk, device=DEV, dtype=torch.int32)
    flag_gems.topk_softmax(w, idx, src, gating.to(DEV), renormalize)
    want_w, want_idx, want_src = O.topk_softmax_ref(gating, topk, renormalize)
    plain_w = O.topk_softmax_ref(gating, topk, False)[0]
    _assert_same_choice(idx.cpu().to(torch.int64), want_idx, plain_w, f"{num_tokens}x{num_experts} top{topk}")
    assert torch.allclose(w.cpu(), want_w, atol=1e-5, rtol=0)
    assert torch.equal(src.cpu(), want_src)
    if renormalize:
        assert torch.allclose(w.sum(dim=-1).cpu(), torch.ones(num_tokens), atol=1e-5)


def test_topk_softmax_ties_strides_and_errors():
    # equal logits: experts 0 .. k-1 at 1 / E each; 16-bit logits tie often and must break to the lower expert
    w = torch.empty(3, 4, device=DEV)
    idx = torch.empty(3, 4, device=DEV, dtype=torch.int32)
    src = torch.empty(3, 4, device=DEV, dtype=torch.int32)
    flag_gems.topk_softmax(w, idx, src, torch.zeros(3, 10, device=DEV), False)
    assert torch.equal(idx.cpu(), torch.arange(4, dtype=torch.int32).expand(3, 4))
    assert torch.allclose(w.cpu(), torch.full((3, 4), 0.1), atol=1e-7)
    g = torch.Generator().manual_seed(1)
    coarse = (torch.randint(-3, 4, (64, 200), generator=g).float() * 0.5).bfloat16()
    w = torch.empty(64, 6, device=DEV)
    idx = torch.empty(64, 6, device=DEV, dtype=torch.int64)
    src = torch.empty(64, 6, device=DEV, dtype=torch.int32)
    wide = torch.zeros(64, 256, dtype=torch.bfloat16, device=DEV)
    wide[:, 8:208] = coarse.to(DEV)
    flag_gems.topk_softmax(w, idx, src, wide[:, 8:208], True)          # a strided view
    want_w, want_idx, _ = O.topk_softmax_ref(coarse, 6, True)
    assert torch.equal(idx.cpu(), want_idx)
    assert torch.allclose(w.cpu(), want_w, atol=1e-6)
    with pytest.raises(TypeError, match="int32/int64/uint32"):
        flag_gems.topk_softmax(w, idx.to(torch.int16), src, wide[:, 8:208])
    with pytest.raises(AssertionError):
        flag_gems.topk_softmax(torch.empty(64, 33, device=DEV), torch.empty(64, 33, device=DEV, dtype=torch.int32),
                               torch.empty(64, 33, device=DEV, dtype=torch.int32), wide[:, 8:208])
    # no tokens
    flag_gems.topk_softmax(w[:0], idx[:0], src[:0], wide[:0, 8:208])


def _tolerance(dtype, scoring_func, renormalize):
    if dtype == torch.bfloat16:
        return 5e-3, 1e-3
    if dtype == torch.float16:
        return (1e-3, 1e-4) if scoring_func == 1 else (5e-3, 1e-3)
    return (5e-4, 1e-4) if renormalize else (1e-5, 1e-5)


def _run_grouped(n_token, n_expert, n_group, topk_group, topk, renormalize, scoring_func, dtype, seed, factor=1.0):
    g = torch.Generator().manual_seed(seed)
    scores = torch.randn(n_token, n_expert, generator=g).to(dtype)
    bias = torch.randn(n_expert, generator=g).to(dtype)
    got_w, got_ids = flag_gems.grouped_topk(scores.to(DEV), n_group, topk_group, topk, renormalize, factor, bias.to(DEV), scoring_func)
    want_w, want_ids = O.grouped_topk_ref(scores, n_group, topk_group, topk, renormalize, factor, bias, scoring_func)
    what = f"T={n_token} E={n_expert} G={n_group} tg={topk_group} k={topk} renorm={renormalize} f={scoring_func} {dtype}"
    assert got_w.dtype == torch.float32 and got_ids.dtype == torch.int32 and got_w.shape == (n_token, topk), what
    if scoring_func == 1 and dtype == torch.float32:
        # the sigmoid of two implementations may differ in the last place: compare the choice by the oracle's own values
        plain = O.grouped_topk_ref(scores, n_group, topk_group, topk, False, 1.0, bias, scoring_func)[0]
        _assert_same_choice(got_ids, want_ids, plain, what, slack=1e-6)
    else:
        assert torch.equal(got_ids.cpu(), want_ids), what
    atol, rtol = _tolerance(dtype, scoring_func, renormalize)
    if torch.equal(got_ids.cpu(), want_ids):
        torch.testing.assert_close(got_w.cpu(), want_w, atol=atol, rtol=rtol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("scoring_func", [0, 1])
@pytest.mark.parametrize("renormalize", [True, False])
@pytest.mark.parametrize("topk", [1, 2])
@pytest.mark.parametrize("n_group", [2, 4])
@pytest.mark.parametrize("n_expert", [8, 16])
@pytest.mark.parametrize("n_token", [1, 3, 8])
def test_grouped_topk_reference_grid(n_token, n_expert, n_group, topk, renormalize, scoring_func, dtype):
    _run_grouped(n_token, n_expert, n_group, topk, topk, renormalize, scoring_func, dtype, 45)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("scoring_func", [0, 1])
@pytest.mark.parametrize("renormalize", [True, False])
@pytest.mark.parametrize("n_token,n_expert,n_group,topk_group,topk", [(32, 64, 8, 2, 8), (64, 64, 8, 2, 8), (200, 256, 8, 4, 8),
                                                                      (17, 384, 12, 3, 6), (5, 1024, 32, 8, 32), (9, 96, 3, 3, 5)])
def test_grouped_topk_larger(n_token, n_expert, n_group, topk_group, topk, renormalize, scoring_func, dtype):
    _run_grouped(n_token, n_expert, n_group, topk_group, topk, renormalize, scoring_func, dtype, 0, factor=2.5)


def test_grouped_topk_ties_special_values_and_errors():
    g = torch.Generator().manual_seed(3)
    # small integers: equal scores everywhere, every sum exact -> bit-equal weights too
    for n_group, per, topk_group, topk in ((1, 4, 1, 2), (2, 4, 1, 3), (4, 3, 2, 4), (4, 2, 3, 5), (8, 8, 4, 8)):
        scores = torch.randint(-2, 3, (50, n_group * per), generator=g).float()
        bias = torch.randint(-1, 2, (n_group * per,), generator=g).float()
        got_w, got_ids = flag_gems.grouped_topk(scores.to(DEV), n_group, topk_group, topk, False, 1.0, bias.to(DEV))
        want_w, want_ids = O.grouped_topk_ref(scores, n_group, topk_group, topk, False, 1.0, bias)
        assert torch.equal(got_ids.cpu(), want_ids) and torch.equal(got_w.cpu(), want_w), (n_group, per)
    # every score -inf: experts 0 .. topk-1 at 1 / topk; groups of one expert take the same fixed answer
    got_w, got_ids = flag_gems.grouped_topk(torch.full((2, 8), float("-inf"), device=DEV), 2, 1, 4, True, 3.0, torch.zeros(8, device=DEV))
    assert torch.equal(got_ids.cpu(), torch.arange(4, dtype=torch.int32).expand(2, 4)) and torch.equal(got_w.cpu(), torch.full((2, 4), 0.25))
    got_w, got_ids = flag_gems.grouped_topk(torch.randn(3, 4, device=DEV), 4, 2, 2, False, 1.0, torch.zeros(4, device=DEV))
    assert torch.equal(got_ids.cpu(), torch.arange(2, dtype=torch.int32).expand(3, 2)) and torch.equal(got_w.cpu(), torch.full((3, 2), 0.5))
    # +inf and NaN group scores count as -inf
    s = torch.tensor([[float("inf"), 1.0, 0.5, 0.25], [float("nan"), 1.0, 0.5, 0.25]])
    got_w, got_ids = flag_gems.grouped_topk(s.to(DEV), 2, 1, 2, False, 1.0, torch.zeros(4, device=DEV))
    assert got_ids.cpu().tolist() == [[2, 3], [2, 3]] and got_w.cpu().tolist() == [[0.5, 0.25], [0.5, 0.25]]
    # a bias of another type and shape is converted like the reference converts it; errors as there
    got = flag_gems.grouped_topk(torch.randn(4, 16, device=DEV).bfloat16(), 4, 2, 2, True, 1.0, torch.zeros(4, 4, device=DEV))
    assert got[0].shape == (4, 2)
    with pytest.raises(ValueError, match="divisible by n_group"):
        flag_gems.grouped_topk(torch.randn(4, 10, device=DEV), 4, 2, 2, True, 1.0, torch.zeros(10, device=DEV))
    with pytest.raises(ValueError, match="scoring_func"):
        flag_gems.grouped_topk(torch.randn(4, 16, device=DEV), 4, 2, 2, True, 1.0, torch.zeros(16, device=DEV), 2)
    with pytest.raises(ValueError, match="bias length"):
        flag_gems.grouped_topk(torch.randn(4, 16, device=DEV), 4, 2, 2, True, 1.0, torch.zeros(8, device=DEV))


def test_vllm_ops_and_the_expert_layer_take_the_routing():
    """_moe_C::topk_softmax / grouped_topk are registered, and their outputs drive fused_experts_impl."""
    flag_gems.patch_empty_vllm()
    g = torch.Generator().manual_seed(8)
    tokens, experts, topk, hidden, inter = 48, 8, 2, 256, 256
    gating = torch.randn(tokens, experts, generator=g)
    w = torch.empty(tokens, topk, device=DEV)
    idx = torch.empty(tokens, topk, device=DEV, dtype=torch.int32)
    src = torch.empty(tokens, topk, device=DEV, dtype=torch.int32)
    torch.ops._moe_C.topk_softmax(w, idx, src, gating.to(DEV), True)
    want_w, want_idx, _ = O.topk_softmax_ref(gating, topk, True)
    assert torch.equal(idx.cpu().long(), want_idx) and torch.allclose(w.cpu(), want_w, atol=1e-5)
    vals, ids = torch.ops._moe_C.grouped_topk(gating.to(DEV), 4, 2, 2, True, 1.0, torch.zeros(experts, device=DEV), 0)
    wv, wi = O.grouped_topk_ref(gating, 4, 2, 2, True, 1.0, torch.zeros(experts))
    assert torch.equal(ids.cpu(), wi) and torch.allclose(vals.cpu(), wv, atol=1e-5)
    # the layer on the routing the operator produced equals the layer on the oracle's routing
    x = torch.randn(tokens, hidden, generator=g).bfloat16()
    w1 = (torch.randn(experts, 2 * inter, hidden, generator=g) * 0.05)
    w2 = (torch.randn(experts, hidden, inter, generator=g) * 0.05)
    q1, s1 = zip(*(O.per_block_cast_to_fp8_ref(w1[e]) for e in range(experts)))
    q2, s2 = zip(*(O.per_block_cast_to_fp8_ref(w2[e]) for e in range(experts)))
    q1, s1, q2, s2 = (torch.stack(t).to(DEV) for t in (q1, s1, q2, s2))
    a = flag_gems.fused_experts_impl(x.to(DEV), q1, q2, w, idx, use_fp8_w8a8=True, w1_scale=s1, w2_scale=s2, block_shape=[128, 128])
    b = flag_gems.fused_experts_impl(x.to(DEV), q1, q2, want_w.to(DEV), want_idx.int().to(DEV), use_fp8_w8a8=True, w1_scale=s1,
                                     w2_scale=s2, block_shape=[128, 128])
    torch.testing.assert_close(a.float(), b.float(), rtol=1e-2, atol=1e-2)
