"""GPU parity of aten::_scaled_mm on operands that are not quantized (bf16, fp16, fp32), against the CPU oracle's
restatement of the reference test's own formula (tests/test_scaled_mm.py:111-124: float64 mm, the two scales, the
bias, one cast).  Floating point: the kernel accumulates in fp32 (MFMA), so the bar is
|got - ref| <= 4e-6 * (|a| @ |b|) * scale_a * scale_b  +  one rounding step of the output type  +  1e-30,
far inside the reference's own tolerance (rtol 1e-3 .. 1.6e-2 by dtype, atol 1e-4 * K)."""
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(M, N, K, dtype, out_dtype, scale_mode, use_bias, seed):
    g = torch.Generator().manual_seed(seed)
    a = (0.25 * torch.randn(M, K, generator=g)).to(dtype)
    b = (0.25 * torch.randn(N, K, generator=g)).to(dtype).t()          # column-major [K, N]
    if scale_mode == "scalar":
        sa, sb = torch.tensor([0.75]), torch.tensor([1.25])
    elif scale_mode == "rowwise_1d":
        sa, sb = torch.rand(M, generator=g) + 0.5, torch.rand(N, generator=g) + 0.5
    else:
        sa, sb = torch.rand(M, 1, generator=g) + 0.5, torch.rand(1, N, generator=g) + 0.5
    bias = (0.25 * torch.randn(N, generator=g)).to(out_dtype or dtype) if use_bias else None
    return a, b, sa, sb, bias


def _check(got, a, b, sa, sb, bias, out_dtype, what):
    want_dtype = out_dtype or a.dtype
    assert got.dtype == want_dtype and got.shape == (a.shape[0], b.shape[1]), what
    ref = O.scaled_mm_ref_postscale(a, b, sa, sb, bias, torch.float64)
    mag = (a.double().abs() @ b.double().abs()) * sa.double().reshape(-1, 1) * sb.double().reshape(1, -1)
    bound = 4e-6 * mag + torch.finfo(want_dtype).eps * ref.abs() + 1e-30
    err = (got.cpu().double() - ref).abs()
    assert bool((err <= bound).all()), f"{what}: worst excess {(err - bound).max().item():.3e} at {(err - bound).argmax().item()}"


CASES = [
    (torch.float16, None, "scalar", False),
    (torch.float16, torch.float32, "rowwise_2d", True),
    (torch.float32, torch.float16, "rowwise_1d", True),
    (torch.float32, None, "rowwise_2d", True),
    (torch.bfloat16, torch.float32, "rowwise_2d", False),
    (torch.bfloat16, None, "rowwise_1d", True),
    (torch.bfloat16, torch.float16, "scalar", True),
]
SHAPES = [(1, 1, 8), (16, 32, 64), (33, 65, 129), (128, 128, 32), (130, 250, 100), (256, 384, 512), (1000, 520, 2048),
          # enough 256 x 256 tiles for most compute units: 16-bit operands with 16-bit results take the persistent kernel
          (2560, 4096, 256), (2500, 4200, 192),
          # up to 128 rows: workgroups of 16 columns whose wavefronts share K, several runs of K steps per wavefront
          (64, 272, 4096), (128, 48, 2088), (17, 16, 8200), (97, 100, 520),
          # 128 rows against a wide matrix: the 128 x 128 tiles again (16-bit operands; fp32 stays with the 16-column workgroups)
          (128, 8192, 2048)]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{str(c[0])[6:]}-{str(c[1])[6:] if c[1] else 'default'}-{c[2]}-bias{int(c[3])}")
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_scaled_mm_matches_the_oracle(case, shape):
    dtype, out_dtype, scale_mode, use_bias = case
    M, N, K = shape
    a, b, sa, sb, bias = _case(M, N, K, dtype, out_dtype, scale_mode, use_bias, M + N + K)
    got = flag_gems.scaled_mm(a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV), bias.to(DEV) if use_bias else None,
                              out_dtype=out_dtype)
    _check(got, a, b, sa, sb, bias, out_dtype, f"{case} {shape}")


def test_out_variant_layouts_and_closed_forms():
    a, b, sa, sb, bias = _case(192, 320, 256, torch.bfloat16, torch.float32, "rowwise_2d", True, 5)
    ad, bd = a.to(DEV), b.to(DEV)
    out = torch.empty(192, 320, dtype=torch.float32, device=DEV)
    res = flag_gems.scaled_mm_out(ad, bd, sa.to(DEV), sb.to(DEV), bias.to(DEV), out_dtype=torch.float32, out=out)
    assert res.data_ptr() == out.data_ptr()
    _check(out, a, b, sa, sb, bias, torch.float32, "out variant")
    # row-major mat2 and a strided self: same values
    wide = torch.zeros(192, 300, dtype=torch.bfloat16, device=DEV)
    wide[:, 11:267] = ad
    res2 = flag_gems.scaled_mm(wide[:, 11:267], bd.contiguous(), sa.to(DEV), sb.to(DEV), bias.to(DEV), out_dtype=torch.float32)
    assert torch.equal(res2, out)
    # identity weights with unit scales copy the activations exactly
    eye = torch.eye(256, dtype=torch.bfloat16, device=DEV)
    one = torch.ones(1, device=DEV)
    assert torch.equal(flag_gems.scaled_mm(ad, eye, one, one), ad)
    # linear in the scales: doubling scale_a doubles every output exactly (powers of two)
    two = flag_gems.scaled_mm(ad, bd, 2 * sa.to(DEV), sb.to(DEV), None, out_dtype=torch.float32)
    base = flag_gems.scaled_mm(ad, bd, sa.to(DEV), sb.to(DEV), None, out_dtype=torch.float32)
    assert torch.equal(two, 2 * base)
    # no K at all: zeros plus the bias
    empty = flag_gems.scaled_mm(ad[:, :0], bd[:0, :], sa.to(DEV), sb.to(DEV), bias.to(DEV), out_dtype=torch.float32)
    assert torch.equal(empty, bias.to(DEV).reshape(1, -1).expand(192, 320))


def test_errors_follow_the_reference():
    a = torch.zeros(4, 8, dtype=torch.bfloat16, device=DEV)
    b = torch.zeros(8, 4, dtype=torch.bfloat16, device=DEV)
    one = torch.ones(1, device=DEV)
    with pytest.raises(RuntimeError, match="same dtype"):
        flag_gems.scaled_mm(a, b.half(), one, one)
    with pytest.raises(RuntimeError, match="cannot be multiplied"):
        flag_gems.scaled_mm(a, b[:4], one, one)
    with pytest.raises(RuntimeError, match="scale_a must be"):
        flag_gems.scaled_mm(a, b, torch.ones(3, device=DEV), one)
    with pytest.raises(RuntimeError, match="Bias must be size"):
        flag_gems.scaled_mm(a, b, one, one, torch.zeros(3, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(NotImplementedError):
        flag_gems.scaled_mm(a.double(), b.double(), one, one)
