"""Pins of the oracle's inverse-RoPE quantizer restatement (CPU only).  Each check compares it with something that does
not share its formula text: answers the rotation's mathematics fixes, a float64 evaluation with complex numbers, exact
cases, the separately pinned per-token-group quantizer, and inputs whose scales and exponent bytes are known in advance."""
import math

import pytest
import torch

from oracle import fp8_linear_oracle as O

HEAD, NOPE, ROPE, GROUP = 512, 448, 64, 128


def _cache(angles: torch.Tensor) -> torch.Tensor:
    """[positions, ROPE / 2] angles -> cos || sin rows"""
    return torch.cat((angles.cos(), angles.sin()), dim=-1).float()


def test_rotating_back_a_vector_at_angle_theta_gives_the_x_axis():
    g = torch.Generator().manual_seed(0)
    theta = torch.rand(5, ROPE // 2, generator=g, dtype=torch.float64) * 6.0 - 3.0
    cache = _cache(theta)
    radius = torch.tensor([1.0, 0.5, 3.0, 7.0]).reshape(1, 4, 1)
    o = torch.zeros(5, 4, HEAD)
    o[:, :, NOPE::2] = (theta.cos().unsqueeze(1) * radius).float()
    o[:, :, NOPE + 1::2] = (theta.sin().unsqueeze(1) * radius).float()
    got = O.inv_rope_ref(o, torch.arange(5), cache, NOPE, ROPE, round_rotated=False)
    # (r cos t, r sin t) rotated back by t is (r, 0); a forward rotation would give (r cos 2t, r sin 2t)
    assert torch.allclose(got[:, :, NOPE::2], radius.expand(5, 4, ROPE // 2), rtol=0, atol=4e-6)
    assert torch.allclose(got[:, :, NOPE + 1::2], torch.zeros(5, 4, ROPE // 2), rtol=0, atol=4e-6)
    assert (theta.sin().abs() > 0.1).any()  # the case does tell the two directions apart
    assert torch.equal(got[:, :, :NOPE], o[:, :, :NOPE])


def test_rotation_against_complex_arithmetic_in_float64():
    g = torch.Generator().manual_seed(1)
    tokens, heads = 6, 3
    theta = torch.rand(40, ROPE // 2, generator=g, dtype=torch.float64) * 100.0
    cache = _cache(theta)
    pos = torch.tensor([0, 39, 7, 7, 21, 3])
    o = torch.randn(tokens, heads, HEAD, generator=g).bfloat16()
    got = O.inv_rope_ref(o, pos, cache, NOPE, ROPE, round_rotated=False)
    z = torch.complex(o[..., NOPE::2].double(), o[..., NOPE + 1::2].double())
    c = cache.double()[pos]
    back = z * torch.complex(c[:, : ROPE // 2], -c[:, ROPE // 2:]).unsqueeze(1)   # z * exp(-i theta), fp32 cos/sin
    assert torch.allclose(got[..., NOPE::2].double(), back.real, rtol=0, atol=1e-6)
    assert torch.allclose(got[..., NOPE + 1::2].double(), back.imag, rtol=0, atol=1e-6)
    assert got.dtype == torch.float32
    # the test helper's form rounds the rotated tail to the input's type and leaves the rest as it was
    rounded = O.inv_rope_ref(o, pos, cache, NOPE, ROPE, round_rotated=True)
    assert rounded.dtype == torch.bfloat16
    assert torch.equal(rounded[..., NOPE:], got[..., NOPE:].bfloat16()) and torch.equal(rounded[..., :NOPE], o[..., :NOPE])


def test_quarter_and_half_turns_are_exact():
    o = torch.arange(2 * HEAD, dtype=torch.float32).reshape(1, 2, HEAD) - 300.0
    half = ROPE // 2
    cache = torch.zeros(3, ROPE)
    cache[0, :half] = 1.0                      # angle 0
    cache[1, half:] = 1.0                      # angle pi/2: cos 0, sin 1
    cache[2, :half] = -1.0                     # angle pi
    e, d = o[..., NOPE::2], o[..., NOPE + 1::2]
    for position, (we, wd) in enumerate(((e, d), (d, -e), (-e, -d))):
        got = O.inv_rope_ref(o, torch.tensor([position]), cache, NOPE, ROPE, round_rotated=False)
        assert torch.equal(got[..., NOPE::2], we) and torch.equal(got[..., NOPE + 1::2], wd), position
        assert torch.equal(got[..., :NOPE], o[..., :NOPE])


@pytest.mark.parametrize("tma", [False, True])
def test_without_rotation_it_is_the_group_quantizer_on_the_regrouped_heads(tma):
    g = torch.Generator().manual_seed(2)
    tokens, groups, hpg = 5, 2, 3
    o = (torch.randn(tokens, groups * hpg, HEAD, generator=g) * 3).bfloat16()
    cache = torch.zeros(4, ROPE)
    cache[:, : ROPE // 2] = 1.0
    codes, scales = O.fused_inv_rope_fp8_quant_ref(o, torch.tensor([0, 1, 2, 3, 1]), cache, groups, hpg, NOPE, ROPE, GROUP,
                                                   tma_aligned_scales=tma)
    # heads g * hpg .. g * hpg + hpg - 1 of a token side by side, quantized per 128 by the separately pinned quantizer
    flat = o.reshape(tokens, groups, hpg * HEAD).contiguous()
    want_q, want_s = O.per_token_group_quant_fp8_ref(flat, GROUP, scale_ue8m0=tma)
    assert torch.equal(codes.view(torch.uint8), want_q.view(torch.uint8))
    if not tma:
        assert torch.equal(scales, want_s)
    else:
        want_e = (want_s.view(torch.int32) >> 23) & 0xFF                       # [tokens, groups, hpg * 4]
        for h in range(hpg):
            for c in range(4):
                assert torch.equal((scales[..., h] >> (8 * c)) & 0xFF, want_e[..., 4 * h + c]), (h, c)


def test_scales_and_exponent_bytes_known_in_advance():
    tokens, groups, hpg = 3, 2, 2
    o = torch.zeros(tokens, groups * hpg, HEAD)
    want_k = torch.zeros(tokens, groups, hpg, 4, dtype=torch.int32)
    for t in range(tokens):
        for h in range(groups * hpg):
            for c in range(4):
                k = (t * 5 + h * 3 + c * 2) % 13 - 6
                o[t, h, c * GROUP + (7 * h + c) % 64] = -448.0 * 2.0 ** k     # the group's largest magnitude
                o[t, h, c * GROUP + 100 - c] = 2.0 ** k                        # -> code of 1.0
                want_k[t, h // hpg, h % hpg, c] = k
    cache = torch.zeros(2, ROPE)
    cache[:, : ROPE // 2] = 1.0
    pos = torch.tensor([1, 0, 1])
    codes, scales = O.fused_inv_rope_fp8_quant_ref(o, pos, cache, groups, hpg, NOPE, ROPE, GROUP)
    assert torch.equal(scales, (2.0 ** want_k.float()).reshape(tokens, groups, hpg * 4))
    codes_f = codes.float().reshape(tokens, groups, hpg, 4, GROUP)
    assert codes_f.min() == -448.0 and codes_f.max() == 1.0
    for h in range(groups * hpg):
        for c in range(4):
            assert torch.all(codes_f[:, h // hpg, h % hpg, c, (7 * h + c) % 64] == -448.0)
            assert torch.all(codes_f[:, h // hpg, h % hpg, c, 100 - c] == 1.0)
    _, packed = O.fused_inv_rope_fp8_quant_ref(o, pos, cache, groups, hpg, NOPE, ROPE, GROUP, tma_aligned_scales=True)
    assert packed.shape == (tokens, groups, hpg) and packed.dtype == torch.int32
    for c in range(4):
        assert torch.equal((packed >> (8 * c)) & 0xFF, want_k[..., c] + 127), c


def test_power_of_two_scales_lie_in_s_2s_and_all_zero_groups_take_the_floor():
    g = torch.Generator().manual_seed(4)
    o = torch.randn(4, 4, HEAD, generator=g).bfloat16()
    o[1, 2, 128:256] = 0                                                        # a group of zeros
    theta = torch.rand(8, ROPE // 2, generator=g, dtype=torch.float64) * 50
    cache, pos = _cache(theta), torch.tensor([3, 0, 7, 5])
    _, plain = O.fused_inv_rope_fp8_quant_ref(o, pos, cache, 2, 2)
    _, packed = O.fused_inv_rope_fp8_quant_ref(o, pos, cache, 2, 2, tma_aligned_scales=True)
    exps = torch.stack([(packed >> (8 * c)) & 0xFF for c in range(4)], dim=-1).reshape(4, 2, 8)
    pow2 = torch.ldexp(torch.ones(()), exps - 127)
    floor = torch.clamp(plain, min=1e-10)
    assert torch.all(pow2 >= floor) and torch.all(pow2 < 2 * floor)
    assert plain[1, 1, 1] == torch.tensor(1e-10) * torch.tensor(1.0 / 448.0)   # token 1, head 2 = group 1, head 0: its group 1
    assert math.isclose(float(pow2[1, 1, 1]), 2.0 ** -33)                        # the power of two at or above 1e-10
