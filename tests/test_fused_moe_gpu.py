"""The block-fp8 expert layer end to end (quantize -> grouped GEMM 1 -> SiLU-and-mul + quantize -> grouped GEMM 2 ->
sum over the top-k slots) against the CPU restatement of the reference's own check
(tests/test_fused_experts_impl.py:604-662, restated in oracle/fp8_linear_oracle.py: block_fp8_moe_ref).

Bars.  The reference compares with rtol 2e-1 and atol max(5e-2, 5 % of the largest result)
(tests/test_fused_experts_impl.py:752-754); every case here must pass that, and a tighter bar on top: rtol 5e-2,
atol 2 % of the largest result.  A chain of two GEMMs with a quantizer between them cannot be held to the single
GEMM's 1e-2: a bf16 rounding of the first GEMM that falls the other way moves an fp8 code of the second operand by
a whole step (6 % of that element).  The steps themselves are tested one by one at their own bars elsewhere
(bit-exact quantizers, GEMM within rtol / atol 1e-2)."""
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn


def _layer(tokens, experts, hidden, inter, topk, seed, zipf=False, randn_scales=False):
    """Inputs as the reference's test makes them (tests/test_fused_experts_impl.py:683-725); generated on the device,
    which is also where the large weights stay."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.randn(tokens, hidden, device=DEV, generator=g).bfloat16()
    w1 = torch.empty(experts, 2 * inter, hidden, device=DEV, dtype=FP8)
    w2 = torch.empty(experts, hidden, inter, device=DEV, dtype=FP8)
    for e in range(experts):
        w1[e] = (torch.randn(2 * inter, hidden, device=DEV, generator=g) / hidden**0.5).to(FP8)
        w2[e] = (torch.randn(hidden, inter, device=DEV, generator=g) / inter**0.5).to(FP8)
    shape1 = (experts, (2 * inter + 127) // 128, hidden // 128)
    shape2 = (experts, (hidden + 127) // 128, inter // 128)
    if randn_scales:  # the reference draws them from N(0, 1): signs and magnitudes of any kind
        s1 = torch.randn(shape1, device=DEV, generator=g)
        s2 = torch.randn(shape2, device=DEV, generator=g)
    else:
        s1 = torch.rand(shape1, device=DEV, generator=g) + 0.5
        s2 = torch.rand(shape2, device=DEV, generator=g) + 0.5
    gate = torch.randn(tokens, experts, device=DEV, generator=g)
    if zipf:  # expert loads skewed by a Zipf(1.1) law over a seeded permutation of the experts
        perm = torch.randperm(experts, device=DEV, generator=g)
        bias = torch.empty(experts, device=DEV)
        bias[perm] = -1.1 * torch.log(torch.arange(1, experts + 1, device=DEV, dtype=torch.float32))
        gate = gate + 3.0 * bias
    tw, ti = torch.topk(torch.softmax(gate, dim=-1), topk, dim=-1)
    tw = (tw / tw.sum(dim=-1, keepdim=True)).bfloat16()
    return x, w1, w2, s1, s2, tw, ti


def _oracle(x, w1, w2, s1, s2, tw, ti, tokens=None, expert_map=None):
    """The CPU oracle on the sampled tokens; only the weights of the experts those tokens use travel to the host."""
    pick = torch.arange(x.shape[0]) if tokens is None else torch.tensor(tokens)
    ids = ti[pick.to(DEV)].cpu()
    local = ids if expert_map is None else expert_map.cpu()[ids]
    used = sorted({int(e) for e in local.reshape(-1).tolist() if e >= 0})
    # compact the expert axis to the used ones
    remap = torch.full((w1.shape[0] + 1,), -1, dtype=torch.int64)
    for i, e in enumerate(used):
        remap[e] = i
    sub = torch.tensor(used, dtype=torch.int64, device=DEV)
    return O.block_fp8_moe_ref(
        x[pick.to(DEV)].cpu(), w1[sub].cpu(), w2[sub].cpu(), s1[sub].cpu(), s2[sub].cpu(), tw[pick.to(DEV)].cpu(),
        remap[local], [128, 128]), pick


def _assert_close(got, want, what):
    got, want = got.float().cpu(), want.float()
    top = float(want.abs().max())
    torch.testing.assert_close(got, want, rtol=2e-1, atol=max(5e-2, 5e-2 * top), msg=lambda m: f"{what} (reference bar): {m}")
    torch.testing.assert_close(got, want, rtol=5e-2, atol=2e-2 * top + 1e-3, msg=lambda m: f"{what} (tighter bar): {m}")


def _run(x, w1, w2, s1, s2, tw, ti, **kw):
    return flag_gems.fused_experts_impl(x, w1, w2, tw, ti, use_fp8_w8a8=True, w1_scale=s1, w2_scale=s2,
                                        block_shape=[128, 128], **kw)


@pytest.mark.parametrize("config", [(1, 8, 128, 256, 2), (4, 8, 128, 256, 2), (16, 8, 256, 512, 2), (32, 8, 128, 256, 4),
                                    (64, 8, 256, 512, 2), (128, 16, 128, 256, 4)])
@pytest.mark.parametrize("randn_scales", [False, True])
def test_reference_configurations(config, randn_scales):
    """The small configurations of the reference's block-wise fp8 test (FUSED_MOE_QUANT_CONFIGS,
    tests/test_fused_experts_impl.py:63-78), every token against the oracle; once with the reference's N(0, 1) weight
    scales."""
    tokens, experts, hidden, inter, topk = config
    args = _layer(tokens, experts, hidden, inter, topk, seed=tokens + experts, randn_scales=randn_scales)
    got = _run(*args)
    assert got.shape == (tokens, hidden) and got.dtype == torch.bfloat16
    want, _ = _oracle(*args)
    _assert_close(got, want, f"config {config}")
    again = _run(*args)
    assert torch.equal(again.view(torch.int16), got.view(torch.int16)), "two runs of one layer differ"
    # the two wrappers of the reference (src/flag_gems/fused/fused_moe.py:2188-2291)
    x, w1, w2, s1, s2, tw, ti = args
    kw = dict(use_fp8_w8a8=True, w1_scale=s1, w2_scale=s2, block_shape=[128, 128])
    assert torch.equal(flag_gems.outplace_fused_experts(x, w1, w2, tw, ti, **kw), got)
    y = x.clone()
    assert flag_gems.inplace_fused_experts(y, w1, w2, tw, ti, **kw) is None
    assert torch.equal(y, got)


@pytest.mark.parametrize("tokens", [1, 16, 64, 1024, 4096])
def test_mixtral_layer_on_sampled_tokens(tokens):
    """Mixtral-8x7B expert layer (8 experts, top-2, hidden 4096, intermediate 14336; the reference's own list has it
    for 1, 16 and 64 tokens, tests/test_fused_experts_impl.py:74-77) with Zipf-skewed expert loads for 64, 1024 and
    4096 tokens: the oracle on a sample of tokens."""
    args = _layer(tokens, 8, 4096, 14336, 2, seed=tokens, zipf=tokens >= 64)
    got = _run(*args)
    sample = sorted({0, 1 % tokens, tokens // 3, tokens // 2, tokens - 2 if tokens > 1 else 0, tokens - 1})
    want, pick = _oracle(*args, tokens=sample)
    _assert_close(got[pick.to(DEV)], want, f"{tokens} tokens")
    assert torch.isfinite(got.float()).all()
    again = _run(*args)
    assert torch.equal(again.view(torch.int16), got.view(torch.int16))


def test_many_experts_few_tokens():
    """16 tokens over 512 experts, top-10 (the Qwen3.5-like shape of the reference's list,
    tests/test_fused_experts_impl.py:85-93): most experts get no row at all."""
    args = _layer(16, 512, 4096, 1024, 10, seed=9)
    got = _run(*args)
    want, pick = _oracle(*args, tokens=[0, 5, 15])
    _assert_close(got[pick.to(DEV)], want, "512 experts")


def test_expert_map_zeroes_slots_of_foreign_experts():
    """Expert parallelism: this rank holds global experts 5, 1 and 6 as its local experts 0, 1 and 2 (so local ids
    are not ascending in global order, and foreign experts lie before, between and after them).  Slots of foreign
    experts contribute zeros (src/flag_gems/fused/fused_moe.py:1114, 2128-2129)."""
    tokens, experts, hidden, inter, topk = 96, 8, 256, 512, 2
    x, w1, w2, s1, s2, tw, ti = _layer(tokens, experts, hidden, inter, topk, seed=21)
    emap = torch.full((experts,), -1, dtype=torch.int64, device=DEV)
    owned = [5, 1, 6]
    for local, g in enumerate(owned):
        emap[g] = local
    sub = torch.tensor(owned, device=DEV)
    got = _run(x, w1[sub].contiguous(), w2[sub].contiguous(), s1[sub].contiguous(), s2[sub].contiguous(), tw, ti,
               expert_map=emap, global_num_experts=experts)
    want = O.block_fp8_moe_ref(x.cpu(), w1[sub].cpu(), w2[sub].cpu(), s1[sub].cpu(), s2[sub].cpu(), tw.cpu(), ti.cpu(),
                               [128, 128], expert_map=emap.cpu())
    _assert_close(got, want, "expert_map")
    foreign = ~torch.isin(ti, sub).any(dim=1)
    assert int(foreign.sum()) > 0, "the case must hold tokens whose experts are all elsewhere"
    assert float(got[foreign].float().abs().max()) == 0.0


def test_moe_align_tables_with_interior_foreign_blocks():
    """The tables of the reference's moe_align_block_size after expert_map (one local expert or -1 per block of
    block_m sorted rows, src/flag_gems/fused/moe_align_block_size.py:771-819): -1 blocks in front of and between the
    local experts' blocks, local ids out of order.  local_rows_from_moe_align reorders the blocks; the GEMM then
    multiplies every row by its own expert's weights and stores zeros for rows of foreign blocks."""
    block_m, N, K, E = 16, 384, 256, 3
    for ids in ([-1, -1, 0, 1, 1, -1], [2, 2, -1, 0, 1, 1, -1]):
        expert_ids = torch.tensor(ids, dtype=torch.int32, device=DEV)
        nb = len(ids)
        tokens = nb * block_m  # every sorted row is a real slot here, so that foreign rows are seen to hold zeros
        g = torch.Generator().manual_seed(nb)
        sorted_token_ids = torch.randperm(tokens, generator=g).to(torch.int32).to(DEV)
        x = torch.randn(tokens, K, generator=g).bfloat16()
        xq, xs = O.act_quant_ref(x, 128)
        wq, ws = [], []
        for _ in range(E):
            q, s = O.per_block_cast_to_fp8_ref((0.02 * torch.randn(N, K, generator=g)).bfloat16())
            wq.append(q); ws.append(s)
        wq, ws = torch.stack(wq), torch.stack(ws)
        rows, offs = flag_gems.local_rows_from_moe_align(sorted_token_ids, expert_ids, block_m, E)
        got = flag_gems.grouped_w8a8_block_fp8_matmul(
            xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), offs, [128, 128], row_index=rows, index_divisor=1,
            scatter_rows=tokens, zero_unwritten_rows=True).cpu().float()
        want = torch.zeros(tokens, N)
        st = sorted_token_ids.cpu().long()
        for b, e in enumerate(ids):
            if e >= 0:
                r = st[b * block_m:(b + 1) * block_m]
                want[r] = O.block_fp8_matmul_tiled_ref(xq[r], wq[e], xs[r], ws[e], [128, 128], torch.float32)
        torch.testing.assert_close(got, want, rtol=1e-2, atol=1e-2, msg=lambda m: f"expert_ids {ids}: {m}")
        for b, e in enumerate(ids):
            if e < 0:
                assert float(got[st[b * block_m:(b + 1) * block_m]].abs().max()) == 0.0


def _sorted_table(ids, experts, emap):
    """The table by definition, on the host: key = local expert or `experts`; a stable sort by key; cumulative counts."""
    flat = ids.reshape(-1).cpu().long()
    if emap is not None:
        m = emap.cpu().long()
        inside = (flat >= 0) & (flat < m.numel())
        flat = torch.where(inside, m[flat.clamp(0, max(m.numel() - 1, 0))], torch.full_like(flat, -1))
    key = torch.where((flat >= 0) & (flat < experts), flat, torch.full_like(flat, experts))
    order = torch.sort(key, stable=True).indices.to(torch.int32)
    offs = torch.cumsum(torch.bincount(key, minlength=experts + 1)[:experts], 0).to(torch.int32)
    return order, offs


@pytest.mark.parametrize("slots", [0, 1, 63, 64, 65, 1000, 1024, 1025, 8192, 32768, 65536, 70000])
@pytest.mark.parametrize("experts", [1, 8, 256, 960, 1000])
def test_moe_sort_slots_is_a_stable_sort_by_expert(slots, experts):
    """The routing table against its definition: every size around the kernel's 1024-slot rounds and its limits
    (65536 slots, 960 experts; beyond them the table comes from torch's sort and must be the same), int32 and int64
    ids, ids that name no expert (-1, too large), an expert_map of either width with foreign experts."""
    g = torch.Generator().manual_seed(slots * 7 + experts)
    for id_dtype, map_dtype in ((torch.int64, None), (torch.int32, torch.int32), (torch.int64, torch.int64), (torch.int32, None)):
        global_experts = experts if map_dtype is None else experts + 5
        ids = torch.randint(-1, global_experts + 2, (slots,), generator=g).to(id_dtype)
        if slots > 100:  # a long run of one expert, and one expert that never occurs
            ids[10:90] = 0
            ids[ids == min(1, global_experts - 1)] = 0
        emap = None
        if map_dtype is not None:
            perm = torch.randperm(global_experts, generator=g)
            emap = torch.full((global_experts,), -1, dtype=map_dtype)
            emap[perm[:experts]] = torch.arange(experts, dtype=map_dtype)
        got_rows, got_offs = flag_gems.moe_sort_slots(ids.to(DEV), experts, None if emap is None else emap.to(DEV))
        want_rows, want_offs = _sorted_table(ids, experts, emap)
        assert got_rows.dtype == torch.int32 and got_offs.dtype == torch.int32
        assert torch.equal(got_offs.cpu(), want_offs), f"offs, {slots} slots, {experts} experts, {id_dtype}, map {map_dtype}"
        assert torch.equal(got_rows.cpu(), want_rows), f"order, {slots} slots, {experts} experts, {id_dtype}, map {map_dtype}"


@pytest.mark.parametrize("slots,experts,block_m", [(0, 4, 16), (0, 3, 1), (1, 1, 16), (130, 8, 16), (1000, 8, 64), (4096, 64, 16), (8192, 8, 128),
                                                   (20000, 256, 64), (65536, 960, 16), (333, 512, 1)])
@pytest.mark.parametrize("pad_sorted_ids", [False, True])
def test_moe_align_block_size_layout(slots, experts, block_m, pad_sorted_ids):
    """The padded table in the reference's format (src/flag_gems/fused/moe_align_block_size.py:771-819) against its
    definition: shapes as the reference allocates them, every expert's slots in ascending order from a block boundary,
    the padding value everywhere else, the expert of every block, the padded length."""
    g = torch.Generator().manual_seed(slots + experts)
    ids = torch.randint(0, experts, (slots,), generator=g)
    if slots > 100:
        ids[ids == experts // 2] = 0  # an expert without slots (when there is more than one)
    for dtype in (torch.int64, torch.int32):
        sorted_ids, expert_ids, post = flag_gems.moe_align_block_size(ids.to(dtype).to(DEV), block_m, experts, pad_sorted_ids=pad_sorted_ids)
        cap = slots + experts * (block_m - 1)
        if pad_sorted_ids:
            cap = -(-cap // block_m) * block_m
        assert sorted_ids.shape == (cap,) and sorted_ids.dtype == torch.int32
        assert expert_ids.shape == (-(-cap // block_m),) and post.shape == (1,)
        counts = torch.bincount(ids, minlength=experts)
        padded = (counts + block_m - 1) // block_m * block_m
        want_sorted = torch.full((cap,), slots, dtype=torch.int32)
        want_blocks = torch.full((-(-cap // block_m),), -1, dtype=torch.int32)
        start = 0
        order = torch.sort(ids, stable=True).indices.to(torch.int32)
        taken = 0
        for e in range(experts):
            c, p = int(counts[e]), int(padded[e])
            want_sorted[start:start + c] = order[taken:taken + c]
            want_blocks[start // block_m:(start + p) // block_m] = e
            start += p
            taken += c
        assert int(post) == start
        assert torch.equal(sorted_ids.cpu(), want_sorted)
        assert torch.equal(expert_ids.cpu(), want_blocks)


def test_moe_align_table_feeds_the_grouped_gemm_under_expert_map():
    """The reference's flow end to end: moe_align_block_size with an expert_map (two local experts out of five, in
    swapped order), local_rows_from_moe_align, the grouped GEMM with scattered rows: every slot of a local expert gets
    its own expert's product, every other slot zeros."""
    tokens, top_k, N, K, block_m = 200, 2, 384, 256, 16
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, 5, (tokens, top_k), generator=g)
    emap = torch.tensor([-1, 1, -1, 0, -1], dtype=torch.int32)  # global 3 -> local 0, global 1 -> local 1
    sorted_ids, expert_ids, _ = flag_gems.moe_align_block_size(ids.to(DEV), block_m, 5, expert_map=emap.to(DEV))
    rows, offs = flag_gems.local_rows_from_moe_align(sorted_ids, expert_ids, block_m, 2)
    x = torch.randn(tokens, K, generator=g).bfloat16()
    xq, xs = O.act_quant_ref(x, 128)
    wq, ws = [], []
    for _ in range(2):
        q, s = O.per_block_cast_to_fp8_ref((0.02 * torch.randn(N, K, generator=g)).bfloat16())
        wq.append(q); ws.append(s)
    wq, ws = torch.stack(wq), torch.stack(ws)
    got = flag_gems.grouped_w8a8_block_fp8_matmul(
        xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), offs, [128, 128], row_index=rows, index_divisor=top_k,
        scatter_rows=tokens * top_k, zero_unwritten_rows=True).cpu().float()
    flat = ids.reshape(-1)
    want = torch.zeros(tokens * top_k, N)
    for local, glob in ((0, 3), (1, 1)):
        slots_e = torch.nonzero(flat == glob).reshape(-1)
        tok = slots_e // top_k
        want[slots_e] = O.block_fp8_matmul_tiled_ref(xq[tok], wq[local], xs[tok], ws[local], [128, 128], torch.float32)
    torch.testing.assert_close(got, want, rtol=1e-2, atol=1e-2)
    foreign = ~((flat == 3) | (flat == 1))
    assert float(got[foreign].abs().max()) == 0.0


def test_vllm_moe_ops_write_the_callers_buffers():
    """``_moe_C::moe_align_block_size`` and ``_moe_C::moe_sum`` as vLLM calls them, with buffers it allocated
    (src/flag_gems/patches/patch_vllm_all.py:306-321, 356-359; schemas of patch_util.py:74-85)."""
    flag_gems.patch_empty_vllm()
    ids = torch.randint(0, 8, (300, 2), generator=torch.Generator().manual_seed(5)).to(DEV)
    block_m = 16
    cap = ids.numel() + 8 * (block_m - 1)
    sorted_ids = torch.empty(cap, dtype=torch.int32, device=DEV)
    expert_ids = torch.empty(-(-cap // block_m), dtype=torch.int32, device=DEV)
    post = torch.empty(1, dtype=torch.int32, device=DEV)
    torch.ops._moe_C.moe_align_block_size(ids, 8, block_m, sorted_ids, expert_ids, post)
    a, b, c = flag_gems.moe_align_block_size(ids, block_m, 8)
    assert torch.equal(sorted_ids, a) and torch.equal(expert_ids, b) and torch.equal(post, c)
    x = torch.randn(40, 2, 256, device=DEV).bfloat16()
    out = torch.empty(40, 256, device=DEV, dtype=torch.bfloat16)
    torch.ops._moe_C.moe_sum(x, out)
    assert torch.equal(out, (x[:, 0].float() + x[:, 1].float()).bfloat16())


def test_expert_layer_under_graph_capture():
    """The layer recorded into a HIP graph on a side stream after a warm-up call (the serving flow) and replayed on
    new inputs written into the captured buffers: every replay equals the eager call on the same inputs.  Nothing
    in the chain synchronises or allocates outside torch's graph pool."""
    tokens, experts, hidden, inter, topk = 48, 8, 512, 1024, 2
    x, w1, w2, s1, s2, tw, ti = _layer(tokens, experts, hidden, inter, topk, seed=77)
    static_x, static_tw, static_ti = x.clone(), tw.clone(), ti.clone()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        _run(static_x, w1, w2, s1, s2, static_tw, static_ti)  # warm-up: workspaces, first-launch work
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            static_out = _run(static_x, w1, w2, s1, s2, static_tw, static_ti)
    torch.cuda.synchronize()
    for seed in (78, 79, 80):
        nx, _, _, _, _, ntw, nti = _layer(tokens, experts, hidden, inter, topk, seed=seed)
        static_x.copy_(nx); static_tw.copy_(ntw); static_ti.copy_(nti)
        graph.replay()
        torch.cuda.synchronize()
        want = _run(nx, w1, w2, s1, s2, ntw, nti)  # eager work between the replays
        assert torch.equal(static_out.view(torch.int16), want.view(torch.int16)), f"replay with seed {seed}"


def test_moe_sum_rounds_once():
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        x = (torch.randn(37, 6, 264, device=DEV) * 3).to(dtype)
        out = torch.empty(37, 264, device=DEV, dtype=dtype)
        flag_gems.moe_sum(x, out)
        acc = torch.zeros(37, 264, device=DEV)
        for k in range(6):  # the reference's loop: fp32 running sum in slot order (src/flag_gems/fused/moe_sum.py:54-60)
            acc += x[:, k].float()
        assert torch.equal(out, acc.to(dtype))
