"""GPU parity of fused_inv_rope_fp8_quant: codes and scales bit for bit against the CPU oracle's restatement of the
reference kernel's arithmetic (fp32 rotation, no intermediate rounding), and the reference's own test battery
(tests/test_fused_inv_rope_fp8_quant.py) against its torch helper, which rounds the rotated values to the input's type
first: scale ratio in [0.5, 2] and 1 - cosine similarity of the dequantized values below 1e-4, as there."""
import math

import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O
from tests._util import assert_codes_equal, assert_scales_equal

pytestmark = pytest.mark.gpu
DEV = "cuda"
HEAD_DIM, NOPE_DIM, ROPE_DIM, GROUP = 512, 448, 64, 128


def _make_cos_sin_cache(max_pos, rope_dim):
    half = rope_dim // 2
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, half, dtype=torch.float32) / half))
    freqs = torch.outer(torch.arange(max_pos, dtype=torch.float32), inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1)


def _yarn_cache(max_pos, rope_dim, scaling_factor=16, base=10000.0, beta_fast=32, beta_slow=1):
    """A YaRN-scaled cache like DeepSeek-V4's (the shape of the reference test's _make_real_deepseek_v4_cache,
    tests/test_fused_inv_rope_fp8_quant.py:224-243): interpolated and extrapolated frequencies blended by a linear ramp."""
    pos_freqs = base ** (torch.arange(0, rope_dim, 2, dtype=torch.float32) / rope_dim)

    def correction_dim(rotations):
        return rope_dim * math.log(max_pos / (rotations * 2 * math.pi)) / (2 * math.log(base))

    low, high = max(math.floor(correction_dim(beta_fast)), 0), min(math.ceil(correction_dim(beta_slow)), rope_dim - 1)
    ramp = ((torch.arange(rope_dim // 2, dtype=torch.float32) - low) / max(high - low, 0.001)).clamp(0, 1)
    mask = 1.0 - ramp
    inv_freq = (1.0 / (scaling_factor * pos_freqs)) * (1 - mask) + (1.0 / pos_freqs) * mask
    freqs = torch.outer(torch.arange(max_pos * scaling_factor, dtype=torch.float32), inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1)


def _unpack(packed, chunks=4):
    """int32 words of exponent bytes -> fp32 powers of two, [..., words * chunks]"""
    p = packed.cpu()
    e = torch.stack([(p >> (8 * c)) & 0xFF for c in range(chunks)], dim=-1)
    return (e << 23).contiguous().view(torch.float32).reshape(*p.shape[:-1], p.shape[-1] * chunks)


def _dequant(codes, scale):
    s = _unpack(scale) if scale.dtype == torch.int32 else scale.cpu()
    c = codes.cpu().float()
    return c * s.unsqueeze(-1).expand(*s.shape, GROUP).reshape(c.shape)


def _one_minus_cosine(a, b):
    a, b = a.flatten().double(), b.flatten().double()
    return 1.0 - float((a @ b) / (a.norm() * b.norm()))


def _case(num_tokens, num_heads, n_groups, tma, seed=0, scale=1.0, positions=None, cache=None, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    max_pos = max(4096, num_tokens * 2)
    o = (scale * torch.randn(num_tokens, num_heads, HEAD_DIM, generator=g)).to(dtype)
    if positions is None:
        positions = torch.randint(0, max_pos, (num_tokens,), generator=g)
    if cache is None:
        cache = _make_cos_sin_cache(max_pos, ROPE_DIM)
    hpg = num_heads // n_groups
    out, sc = flag_gems.fused_inv_rope_fp8_quant(o.to(DEV), positions.to(DEV), cache.to(DEV), n_groups, hpg, tma_aligned_scales=tma)
    return dict(o=o, positions=positions, cache=cache, out=out, scale=sc, hpg=hpg, n_groups=n_groups, tma=tma)


def _check_bits(r, what):
    want_q, want_s = O.fused_inv_rope_fp8_quant_ref(r["o"], r["positions"], r["cache"], r["n_groups"], r["hpg"],
                                                    tma_aligned_scales=r["tma"])
    assert_codes_equal(r["out"], want_q, what)
    if r["tma"]:
        assert torch.equal(r["scale"].cpu(), want_s), what
    else:
        assert_scales_equal(r["scale"], want_s, what)


def _check_reference_bars(r, what):
    ref_q, ref_s = O.fused_inv_rope_fp8_quant_ref(r["o"], r["positions"], r["cache"], r["n_groups"], r["hpg"],
                                                  tma_aligned_scales=r["tma"], round_rotated=True)
    got_s = _unpack(r["scale"]) if r["tma"] else r["scale"].cpu()
    want_s = _unpack(ref_s) if r["tma"] else ref_s
    ratio = got_s / want_s.clamp(min=1e-30)
    assert ratio.max() <= 2.0 and ratio.min() >= 0.5, what
    assert _one_minus_cosine(_dequant(r["out"], r["scale"]), _dequant(ref_q, ref_s)) < 1e-4, what


@pytest.mark.parametrize("seed", [0, 42])
@pytest.mark.parametrize("tma", [False, True])
@pytest.mark.parametrize("num_heads,n_groups", [(32, 4), (64, 8), (128, 8)])
@pytest.mark.parametrize("num_tokens", [1, 7, 32, 128])
def test_reference_grid(num_tokens, num_heads, n_groups, tma, seed):
    r = _case(num_tokens, num_heads, n_groups, tma, seed=seed)
    what = f"T={num_tokens} H={num_heads} G={n_groups} tma={tma} seed={seed}"
    _check_bits(r, what)
    _check_reference_bars(r, what)


@pytest.mark.parametrize("num_heads,n_groups", [(64, 8), (128, 8)])
@pytest.mark.parametrize("num_tokens", [1, 7, 32, 128])
def test_output_layout(num_tokens, num_heads, n_groups):
    d = (num_heads // n_groups) * HEAD_DIM
    plain = _case(num_tokens, num_heads, n_groups, False)
    assert plain["out"].shape == (num_tokens, n_groups, d) and plain["out"].stride() == (d, num_tokens * d, 1)
    assert plain["scale"].shape == (num_tokens, n_groups, d // GROUP) and plain["scale"].dtype == torch.float32
    assert plain["scale"].permute(1, 0, 2).stride(1) == 1 or num_tokens == 1
    packed = _case(num_tokens, num_heads, n_groups, True)
    assert packed["out"].stride() == (d, num_tokens * d, 1)
    assert packed["scale"].dtype == torch.int32 and packed["scale"].shape[-1] == (d // GROUP + 3) // 4
    assert packed["scale"].permute(1, 0, 2).stride(1) == 1 or num_tokens == 1
    for g in range(n_groups):
        assert plain["out"][:, g, :].is_contiguous()
    # the rows that pad the token count to a multiple of four read as zero scales
    padded = (num_tokens + 3) // 4 * 4
    for r in (plain, packed):
        inner = r["scale"].shape[-1]
        raw = torch.as_strided(r["scale"], (n_groups, inner, padded), (inner * padded, padded, 1))
        assert torch.all(raw[:, :, num_tokens:] == 0)


@pytest.mark.parametrize("tma", [False, True])
def test_scales_are_powers_of_two_only_when_packed(tma):
    r = _case(32, 64, 8, tma)
    s = _unpack(r["scale"]) if tma else r["scale"].cpu()
    residual = (torch.log2(s) - torch.log2(s).round()).abs().max()
    assert (residual < 1e-5) if tma else (residual > 1e-5)


@pytest.mark.parametrize("tma", [False, True])
def test_large_values_zero_positions_and_a_yarn_cache(tma):
    r = _case(8, 64, 8, tma, scale=1000.0)
    _check_bits(r, "large")
    _check_reference_bars(r, "large")
    r = _case(16, 64, 8, tma, positions=torch.zeros(16, dtype=torch.long))
    _check_bits(r, "zero positions")
    assert_codes_equal(r["out"], O.per_token_group_quant_fp8_ref(r["o"].reshape(16, 8, 8 * HEAD_DIM), GROUP, scale_ue8m0=tma)[0],
                       "position 0 rotates nothing")
    cache = _yarn_cache(4096, ROPE_DIM)
    for tokens in (1, 32, 256):
        g = torch.Generator().manual_seed(tokens)
        r = _case(tokens, 64, 8, tma, positions=torch.randint(0, 4096, (tokens,), generator=g), cache=cache)
        _check_bits(r, f"yarn {tokens}")
        _check_reference_bars(r, f"yarn {tokens}")


@pytest.mark.parametrize("tma", [False, True])
def test_nope_dims_do_not_depend_on_the_rotation(tma):
    r = _case(16, 64, 8, tma)
    still = torch.zeros_like(r["cache"])
    still[:, : ROPE_DIM // 2] = 1.0
    n = _case(16, 64, 8, tma, positions=r["positions"], cache=still)
    s1 = _unpack(r["scale"]) if tma else r["scale"].cpu()
    s2 = _unpack(n["scale"]) if tma else n["scale"].cpu()
    for h in range(8):
        for c in range(3):
            qb = h * 4 + c
            a = r["out"][:, :, qb * GROUP:(qb + 1) * GROUP].cpu().view(torch.uint8)
            b = n["out"][:, :, qb * GROUP:(qb + 1) * GROUP].cpu().view(torch.uint8)
            assert torch.equal(a, b) and torch.equal(s1[:, :, qb], s2[:, :, qb]), (h, c)


def test_dequantized_values_are_close_to_the_rotated_input():
    r = _case(32, 64, 8, False)
    rotated = O.inv_rope_ref(r["o"], r["positions"], r["cache"], NOPE_DIM, ROPE_DIM).reshape(32, 8, 8 * HEAD_DIM).float()
    rel = (_dequant(r["out"], r["scale"]) - rotated).abs() / rotated.abs().clamp(min=1e-6)
    assert rel.mean() < 0.15


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_other_input_types_int32_positions_and_strided_heads(dtype):
    g = torch.Generator().manual_seed(11)
    tokens, heads, groups = 9, 12, 3
    cache = _make_cos_sin_cache(64, ROPE_DIM)
    pos = torch.randint(0, 64, (tokens,), generator=g)
    wide = (torch.randn(tokens, heads + 2, HEAD_DIM + 64, generator=g) * 2).to(dtype)
    o = wide[:, 1:heads + 1, 32:32 + HEAD_DIM]                       # token, head and element offsets
    for tma in (False, True):
        out, sc = flag_gems.fused_inv_rope_fp8_quant(wide.to(DEV)[:, 1:heads + 1, 32:32 + HEAD_DIM], pos.to(DEV).int(),
                                                     cache.to(DEV), groups, heads // groups, tma_aligned_scales=tma)
        want_q, want_s = O.fused_inv_rope_fp8_quant_ref(o, pos, cache, groups, heads // groups, tma_aligned_scales=tma)
        assert_codes_equal(out, want_q, f"{dtype} tma={tma}")
        assert torch.equal(sc.cpu().view(torch.int32), want_s.view(torch.int32))


@pytest.mark.parametrize("head_dim,rope_dim,group", [(256, 64, 128), (256, 32, 64), (1024, 128, 256), (1536, 64, 512), (128, 128, 128)])
def test_other_head_and_group_sizes(head_dim, rope_dim, group):
    g = torch.Generator().manual_seed(head_dim + group)
    tokens, heads, groups = 6, 10, 2
    cache = _make_cos_sin_cache(32, rope_dim)
    pos = torch.randint(0, 32, (tokens,), generator=g)
    o = torch.randn(tokens, heads, head_dim, generator=g).bfloat16()
    out, sc = flag_gems.fused_inv_rope_fp8_quant(o.to(DEV), pos.to(DEV), cache.to(DEV), groups, heads // groups,
                                                 nope_dim=head_dim - rope_dim, rope_dim=rope_dim, quant_group_size=group)
    want_q, want_s = O.fused_inv_rope_fp8_quant_ref(o, pos, cache, groups, heads // groups, head_dim - rope_dim, rope_dim, group)
    assert_codes_equal(out, want_q, "codes")
    assert_scales_equal(sc, want_s, "scales")


def test_special_values_edges_and_errors():
    cache = _make_cos_sin_cache(16, ROPE_DIM)
    o = torch.randn(4, 8, HEAD_DIM, generator=torch.Generator().manual_seed(5)).bfloat16()
    o[0, 0, :128] = 0                       # an all-zero group: the floor sets the scale
    o[1, 3, 200] = float("inf")
    o[2, 5, 460] = float("nan")             # inside the rotated tail: its partner becomes NaN too
    o[3, 7, 511] = -3e38
    pos = torch.tensor([3, 15, 0, 9])
    for tma in (False, True):
        out, sc = flag_gems.fused_inv_rope_fp8_quant(o.to(DEV), pos.to(DEV), cache.to(DEV), 2, 4, tma_aligned_scales=tma)
        want_q, want_s = O.fused_inv_rope_fp8_quant_ref(o, pos, cache, 2, 4, tma_aligned_scales=tma)
        assert_codes_equal(out, want_q, f"special tma={tma}")
        if tma:
            assert torch.equal(sc.cpu(), want_s)
        else:
            assert_scales_equal(sc, want_s, "special")
    # positions outside the cache read its nearest row instead of memory outside it
    out, _ = flag_gems.fused_inv_rope_fp8_quant(o.to(DEV), torch.tensor([-5, 99, 0, 16]).to(DEV), cache.to(DEV), 2, 4)
    want, _ = O.fused_inv_rope_fp8_quant_ref(o, torch.tensor([0, 15, 0, 15]), cache, 2, 4)
    assert_codes_equal(out, want, "clamped positions")
    # no tokens
    out, sc = flag_gems.fused_inv_rope_fp8_quant(o[:0].to(DEV), pos[:0].to(DEV), cache.to(DEV), 2, 4)
    assert out.shape == (0, 2, 4 * HEAD_DIM) and sc.shape == (0, 2, 16)
    with pytest.raises(AssertionError, match="token count mismatch"):
        flag_gems.fused_inv_rope_fp8_quant(o.to(DEV), pos[:3].to(DEV), cache.to(DEV), 2, 4)
    with pytest.raises(AssertionError):
        flag_gems.fused_inv_rope_fp8_quant(o.to(DEV), pos.to(DEV), cache.to(DEV), 3, 4)
    with pytest.raises(AssertionError):
        flag_gems.fused_inv_rope_fp8_quant(o.to(DEV), pos.to(DEV), cache.to(DEV).double(), 2, 4)
    with pytest.raises(NotImplementedError):
        flag_gems.fused_inv_rope_fp8_quant(o.to(DEV).double(), pos.to(DEV), cache.to(DEV), 2, 4)


def test_the_einsum_reads_the_quantized_heads_in_place():
    """The producer's layout is the grouped output projection's operand: per group a contiguous [tokens, K] matrix
    with scales of unit stride along the tokens."""
    g = torch.Generator().manual_seed(21)
    tokens, groups, hpg, d_out = 96, 4, 2, 384
    k = hpg * HEAD_DIM
    cache = _make_cos_sin_cache(512, ROPE_DIM)
    pos = torch.randint(0, 512, (tokens,), generator=g)
    o = torch.randn(tokens, groups * hpg, HEAD_DIM, generator=g).bfloat16()
    w = torch.randn(groups, d_out, k, generator=g) * 0.05
    wq, ws = O.per_block_cast_to_fp8_ref(w.reshape(groups * d_out, k))
    wq, ws = wq.reshape(groups, d_out, k), ws.reshape(groups, d_out // 128, k // 128)
    xq, xs = flag_gems.fused_inv_rope_fp8_quant(o.to(DEV), pos.to(DEV), cache.to(DEV), groups, hpg)
    got = flag_gems.fp8_einsum("bhr,hdr->bhd", xq, xs, wq.to(DEV), ws.to(DEV))
    want_q, want_s = O.fused_inv_rope_fp8_quant_ref(o, pos, cache, groups, hpg)
    want = O.fp8_block_einsum_ref(want_q, want_s, wq, ws, [128, 128])
    torch.testing.assert_close(got.float().cpu(), want.float(), rtol=1e-2, atol=1e-2)


def test_benchmark_size_by_sample_and_property():
    """4096 tokens x 128 heads (the reference benchmark's largest shape): sampled tokens bit for bit against the oracle,
    and over the whole output the property that a group's largest magnitude encodes to +-448."""
    g = torch.Generator().manual_seed(9)
    tokens, heads, groups = 4096, 128, 8
    cache = _make_cos_sin_cache(8192, ROPE_DIM)
    pos = torch.randint(0, 8192, (tokens,), generator=g)
    o = torch.randn(tokens, heads, HEAD_DIM, generator=g, dtype=torch.float32).bfloat16()
    out, sc = flag_gems.fused_inv_rope_fp8_quant(o.to(DEV), pos.to(DEV), cache.to(DEV), groups, heads // groups)
    pick = torch.tensor([0, 1, 2, 3, 777, 2048, 4093, 4094, 4095])
    want_q, want_s = O.fused_inv_rope_fp8_quant_ref(o[pick], pos[pick], cache, groups, heads // groups)
    assert_codes_equal(out[pick.to(DEV)], want_q, "sample")
    assert_scales_equal(sc[pick.to(DEV)], want_s, "sample")
    top = out.view(torch.uint8).reshape(tokens, groups, -1, GROUP).bitwise_and(0x7F).amax(dim=-1)
    assert bool((top == 0x7E).all())
