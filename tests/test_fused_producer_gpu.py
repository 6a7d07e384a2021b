"""GPU parity of the activation fused into the quantizer (SiLU-and-mul -> per-token-group FP8).

Two bars.  (1) Bit-exact: the fused call gives the codes and scales of the two separate calls (activation stored
in the input's type, then quantized), for every dtype, group size and rule.  (2) Floating point: the activation
against the CPU oracle, which restates the reference's kernel (src/flag_gems/fused/silu_and_mul.py:13-18): the two
sides evaluate exp with different libraries, so a result may land on the other side of a rounding boundary;
tolerance for bf16 / fp16: every element within one step of the output type, and fewer than 1 in 1000 elements
differ at all; for fp32: rtol 1e-6."""
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O
from tests._util import assert_codes_equal, assert_scales_equal

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _x(shape, seed, dtype=torch.bfloat16, scale=2.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 256), (83, 1024), (2048, 7168), (5, 7, 512)])
def test_activation_matches_oracle_within_one_step(dtype, shape):
    x = _x(shape, 0, dtype)
    want = O.silu_and_mul_ref(x)
    got = flag_gems.silu_and_mul_packed(x.to(DEV)).cpu()
    assert got.dtype == dtype and got.shape == want.shape
    if dtype == torch.float32:  # no rounding to a narrower type hides the last bits of exp: a few fp32 steps
        torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-37)
        return
    eps = torch.finfo(dtype).eps
    diff = (got.double() - want.double()).abs()
    assert torch.all(diff <= want.double().abs() * eps + 1e-37)
    assert (got != want).float().mean().item() < 1e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("group", [64, 128])
@pytest.mark.parametrize("ue8m0", [False, True])
def test_fused_equals_the_two_separate_calls(dtype, group, ue8m0):
    for shape, seed in (((300, 2048), 1), ((4096, 1024), 2), ((3, 5, 512), 3)):
        x = _x(shape, seed, dtype, scale=4.0).to(DEV)
        act = flag_gems.silu_and_mul_packed(x)
        want_q, want_s = flag_gems.per_token_group_quant_fp8(act, group, scale_ue8m0=ue8m0)
        q, s = flag_gems.silu_and_mul_per_token_group_quant_fp8(x, group, scale_ue8m0=ue8m0)
        assert q.shape == want_q.shape and s.shape == want_s.shape
        assert_scales_equal(s, want_s, f"{shape}")
        assert_codes_equal(q, want_q, f"{shape}")


def test_fused_rules_layouts_and_special_values():
    x = _x((512, 1024), 4).to(DEV)
    x[0, :512] = 0.0                      # a row of zero gates: every group comes from the floor
    x[1, 5] = float("nan")
    x[2, 700] = float("inf")             # an infinite up value
    x[3, 9] = -200.0                      # a gate for which exp overflows: the activation is -0
    act = flag_gems.silu_and_mul_packed(x)
    for kwargs in ({"column_major_scales": True}, {"scale_rule": "div"}, {"eps": 1e-4}, {"dtype": torch.float8_e5m2}):
        want_q, want_s = flag_gems.per_token_group_quant_fp8(act, 128, **kwargs)
        q, s = flag_gems.silu_and_mul_per_token_group_quant_fp8(x, 128, **kwargs)
        assert s.stride() == want_s.stride()
        assert_scales_equal(s, want_s, str(kwargs))
        assert_codes_equal(q, want_q, str(kwargs))
    # a strided input: the two halves of each row lie inside a wider buffer
    wide = _x((100, 1536), 5).to(DEV)
    view = wide[:, 256:1280]
    want_q, want_s = flag_gems.per_token_group_quant_fp8(flag_gems.silu_and_mul_packed(view), 128)
    q, s = flag_gems.silu_and_mul_per_token_group_quant_fp8(view, 128)
    assert_scales_equal(s, want_s)
    assert_codes_equal(q, want_q)


def test_fused_against_the_oracle_chain():
    """Against activation and quantizer of the oracle: scales within one step of the activation's type, and the
    dequantised values within one code step of each other."""
    x = _x((256, 4096), 6)
    act = O.silu_and_mul_ref(x)
    want_q, want_s = O.per_token_group_quant_fp8_ref(act, 128)
    q, s = flag_gems.silu_and_mul_per_token_group_quant_fp8(x.to(DEV), 128)
    torch.testing.assert_close(s.cpu(), want_s, rtol=2.0 ** -7, atol=0)
    assert (s.cpu() != want_s).float().mean().item() < 1e-2
    deq, want_deq = q.cpu().float().view(256, 16, 128) * s.cpu()[..., None], want_q.float().view(256, 16, 128) * want_s[..., None]
    assert torch.all((deq - want_deq).abs() <= want_s[..., None] * 32 + 1e-30)  # the coarsest e4m3 step is 32 codes
    assert (q.cpu().view(torch.uint8) != want_q.view(torch.uint8)).float().mean().item() < 1e-2


def test_unsupported_requests_fail_loudly():
    x = _x((8, 512), 7).to(DEV)
    with pytest.raises(NotImplementedError):
        flag_gems.silu_and_mul_per_token_group_quant_fp8(x, 32)       # group sizes other than 64 and 128
    with pytest.raises(AssertionError):
        flag_gems.silu_and_mul_per_token_group_quant_fp8(x, 100)
    with pytest.raises(NotImplementedError):
        flag_gems.silu_and_mul_per_token_group_quant_fp8(x[:, 4:260], 64)  # halves that are not 16-byte aligned
    q, s = flag_gems.silu_and_mul_per_token_group_quant_fp8(x[:0], 128)
    assert q.shape == (0, 256) and s.shape == (0, 2)
