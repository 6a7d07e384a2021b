"""Pins of the oracle's routing restatements (CPU only): library routines, closed forms, the published DeepSeek-V3
routing in a different algorithm text, and a pure-Python loop on tiny inputs."""
import pytest
import torch

from oracle import fp8_linear_oracle as O


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens,experts,topk", [(1, 4, 2), (8, 16, 4), (33, 64, 8), (50, 255, 30), (16, 512, 32)])
def test_topk_softmax_against_library_softmax_and_topk(tokens, experts, topk, dtype):
    g = torch.Generator().manual_seed(tokens * 1000 + experts)
    # distinct logits in every row (a shuffled ramp plus noise below the ramp's step): no ties for either routine to break
    ramp = torch.stack([torch.randperm(experts, generator=g) for _ in range(tokens)]).float() * 0.125 - 6.0
    gating = (ramp + 0.01 * torch.rand(tokens, experts, generator=g)).to(dtype)
    if dtype == torch.bfloat16:
        gating = (2 * ramp - 52.0).to(dtype)   # multiples of 1/4 inside [-64, 64) are exact in bf16 and distinct
        assert torch.equal(gating.float(), 2 * ramp - 52.0)
    w, idx, src = O.topk_softmax_ref(gating, topk)
    lib_w, lib_idx = torch.topk(torch.softmax(gating.float(), dim=1), topk, dim=1)
    assert torch.equal(idx, lib_idx)
    assert torch.allclose(w, lib_w, rtol=1e-5, atol=1e-7)
    assert torch.equal(src, (torch.arange(topk).unsqueeze(0) * tokens + torch.arange(tokens).unsqueeze(1)).int())
    wn, idxn, _ = O.topk_softmax_ref(gating, topk, renormalize=True)
    assert torch.equal(idxn, idx)
    assert torch.allclose(wn.sum(1), torch.ones(tokens), atol=1e-6)
    assert torch.allclose(wn, lib_w / lib_w.sum(1, keepdim=True), rtol=1e-5, atol=1e-7)


def test_topk_softmax_ties_and_extremes():
    w, idx, _ = O.topk_softmax_ref(torch.zeros(3, 10), 4)
    assert torch.equal(idx, torch.arange(4).expand(3, 4)) and torch.allclose(w, torch.full((3, 4), 0.1), atol=1e-7)
    # one dominant logit: probability 1, the rest underflow to 0 and come in index order
    x = torch.full((1, 6), -200.0)
    x[0, 4] = 50.0
    w, idx, _ = O.topk_softmax_ref(x, 3)
    assert idx.tolist() == [[4, 0, 1]] and w.tolist() == [[1.0, 0.0, 0.0]]
    # two equal maxima: the lower expert first
    x = torch.tensor([[0.0, 2.0, 1.0, 2.0]])
    assert O.topk_softmax_ref(x, 3)[1].tolist() == [[1, 3, 2]]


def _deepseek_v3_routing(scores, bias, n_group, topk_group, topk, renormalize, factor):
    """The published DeepSeek-V3 gate (masks and library top-k): fp32 throughout."""
    tokens, experts = scores.shape
    choice = scores + bias
    group_scores = choice.view(tokens, n_group, -1).topk(2, dim=-1).values.sum(dim=-1)
    group_idx = torch.topk(group_scores, topk_group, dim=-1, sorted=False).indices
    group_mask = torch.zeros_like(group_scores).scatter_(1, group_idx, 1)
    score_mask = group_mask.unsqueeze(-1).expand(tokens, n_group, experts // n_group).reshape(tokens, experts)
    masked = choice.masked_fill(~score_mask.bool(), float("-inf"))
    ids = torch.topk(masked, topk, dim=-1, sorted=True).indices
    weights = scores.gather(1, ids)
    if renormalize:
        weights = weights / (weights.sum(dim=-1, keepdim=True) + 1e-20)
    return weights * factor, ids


@pytest.mark.parametrize("scoring", [0, 1])
@pytest.mark.parametrize("renormalize", [False, True])
@pytest.mark.parametrize("tokens,experts,n_group,topk_group,topk", [(5, 16, 4, 2, 2), (9, 64, 8, 2, 8), (4, 256, 8, 4, 8), (3, 8, 2, 1, 1)])
def test_grouped_topk_against_the_published_routing(tokens, experts, n_group, topk_group, topk, renormalize, scoring):
    g = torch.Generator().manual_seed(experts + topk + scoring)
    scores = torch.randn(tokens, experts, generator=g)        # fp32 random values: no ties
    bias = torch.randn(experts, generator=g) * 0.1
    vals, ids = O.grouped_topk_ref(scores, n_group, topk_group, topk, renormalize, 2.5, bias, scoring)
    s = torch.sigmoid(scores) if scoring else scores
    want_v, want_i = _deepseek_v3_routing(s, bias, n_group, topk_group, topk, renormalize, 2.5)
    assert torch.equal(ids.long(), want_i)
    assert torch.allclose(vals, want_v, rtol=2e-6, atol=1e-7)
    if renormalize:
        assert torch.allclose(vals.sum(1), torch.full((tokens,), 2.5), rtol=1e-5)


def _by_hand(scores, bias, n_group, topk_group, topk):
    """Lists and sorted(): group score = two largest biased scores; best groups then best experts, ties to the lower index."""
    experts = len(scores)
    per = experts // n_group
    sb = [scores[e] + bias[e] for e in range(experts)]
    gscore = []
    for gi in range(n_group):
        top = sorted(sb[gi * per:(gi + 1) * per], reverse=True)
        gscore.append(top[0] + (top[1] if per > 1 else float("-inf")))
    if max(gscore) == float("-inf"):   # (groups of one expert have no second score: the reference's fixed answer)
        return list(range(topk)), [1.0 / topk] * topk
    groups = sorted(range(n_group), key=lambda gi: (-gscore[gi], gi))[:topk_group]
    cand = [e for e in range(experts) if e // per in groups]
    picked = sorted(cand, key=lambda e: (-sb[e], e))[:topk]
    return picked, [scores[e] for e in picked]


def test_grouped_topk_with_ties_against_a_loop_over_lists():
    g = torch.Generator().manual_seed(3)
    for trial in range(40):
        n_group = [1, 2, 4][trial % 3]
        per = [1, 2, 4, 3][trial % 4]
        experts = n_group * per
        topk_group = 1 + trial % n_group
        topk = 1 + trial % min(4, topk_group * per)
        # small integers: many equal scores, every sum exact
        scores = torch.randint(-2, 3, (6, experts), generator=g).float()
        bias = torch.randint(-1, 2, (experts,), generator=g).float()
        vals, ids = O.grouped_topk_ref(scores, n_group, topk_group, topk, False, 1.0, bias)
        for t in range(6):
            want_ids, want_vals = _by_hand(scores[t].tolist(), bias.tolist(), n_group, topk_group, topk)
            assert ids[t].tolist() == want_ids and vals[t].tolist() == want_vals, (trial, t)


def test_grouped_topk_special_cases():
    g = torch.Generator().manual_seed(5)
    scores = torch.randn(7, 12, generator=g).bfloat16()
    bias = torch.randn(12, generator=g).bfloat16()
    # one group: the plain top-k of score + bias (in bf16), weights = the scores themselves
    vals, ids = O.grouped_topk_ref(scores, 1, 1, 3, False, 1.0, bias)
    want = torch.topk((scores + bias).float(), 3, dim=1).indices
    assert torch.equal(ids.long(), want) and torch.equal(vals, scores.float().gather(1, want))
    # every score -inf: experts 0 .. topk-1 at 1 / topk
    vals, ids = O.grouped_topk_ref(torch.full((2, 8), float("-inf")), 2, 1, 4, True, 3.0, torch.zeros(8))
    assert torch.equal(ids, torch.arange(4, dtype=torch.int32).expand(2, 4)) and torch.equal(vals, torch.full((2, 4), 0.25))
    # a group whose score is +inf or NaN counts as -inf: the other group wins
    s = torch.tensor([[float("inf"), 1.0, 0.5, 0.25], [float("nan"), 1.0, 0.5, 0.25]])
    vals, ids = O.grouped_topk_ref(s, 2, 1, 2, False, 1.0, torch.zeros(4))
    assert ids.tolist() == [[2, 3], [2, 3]] and vals.tolist() == [[0.5, 0.25], [0.5, 0.25]]
