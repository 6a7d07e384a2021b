"""Pins of the oracle's RMSNorm restatements (CPU only): each check compares them with something that does not
share their formula text: a float64 evaluation, torch's own rms_norm, exact integer sums, closed forms and an
exact invariance."""
import numpy as np
import pytest
import torch

from oracle import fp8_linear_oracle as O


def _step(exact: torch.Tensor, dtype) -> torch.Tensor:
    """An upper bound of the spacing of `dtype` around |exact| (the subnormal spacing where that is larger)."""
    fi = torch.finfo(dtype)
    return torch.clamp(exact.abs() * fi.eps, min=2 * fi.smallest_normal * fi.eps)


@pytest.mark.parametrize("cols", [8, 128, 2048, 2056, 7168, 16384])
def test_sum_of_squares_is_exact_on_small_integers_and_close_otherwise(cols):
    g = torch.Generator().manual_seed(cols)
    # integers in [-7, 7]: every partial sum is an integer below 2^24, so any order of exact operations gives the exact
    # sum, while a dropped, repeated or misplaced element changes it
    t = torch.randint(-7, 8, (5, cols), generator=g).float()
    t[0] = 0.0
    t[1, :] = 0.0
    t[1, cols - 1] = 3.0           # only the last element
    t[2, :] = 0.0
    t[2, 0] = 2.0                  # only the first
    want = (t.double() ** 2).sum(1)
    assert torch.equal(O.row_sum_of_squares_f32(t).double(), want)
    assert want[1] == 9 and want[2] == 4
    # every column counted exactly once: one-hot rows
    eye = torch.zeros((cols, cols))
    eye[torch.arange(cols), torch.arange(cols)] = torch.arange(1, cols + 1, dtype=torch.float32) % 5 + 1
    assert torch.equal(O.row_sum_of_squares_f32(eye), (torch.arange(1, cols + 1, dtype=torch.float32) % 5 + 1) ** 2)
    # random data: within the bound of a pairwise-ish fp32 summation of the exact sum
    x = torch.randn((16, cols), generator=g)
    got = O.row_sum_of_squares_f32(x).double()
    exact = (x.double() ** 2).sum(1)
    assert torch.all((got - exact).abs() <= exact * (cols // 256 + 20) * 2.0 ** -24)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_rms_norm_ref_pinned(dtype):
    g = torch.Generator().manual_seed(3)
    rows, cols, eps = 24, 1536, 1e-5
    x = (2 * torch.randn(rows, cols, generator=g)).to(dtype)
    w = (1 + 0.2 * torch.randn(cols, generator=g)).to(dtype)
    got = O.rms_norm_ref(x, w, eps)
    assert got.dtype == dtype and got.shape == x.shape
    xd, wd = x.double(), w.double()
    exact_n = xd / torch.sqrt((xd * xd).mean(1, keepdim=True) + eps)
    exact = exact_n * wd
    # two roundings to the dtype (the normalised value, then the product): at most one step off in all, plus the
    # fp32 noise of the variance (a few 2^-24)
    assert torch.all((got.double() - exact).abs() <= 1.01 * _step(exact, dtype) + 1e-6 * exact.abs() + 1e-30)
    # a library routine for the same function (fp32 arithmetic, one rounding at the end)
    lib = torch.nn.functional.rms_norm(x.float(), (cols,), w.float(), eps)
    torch.testing.assert_close(got.float(), lib, rtol=2.1 * torch.finfo(dtype).eps + 1e-6, atol=1e-30)
    # rows of one repeated value c: y = w * c / sqrt(c^2 + eps)
    c = torch.tensor([0.5, -3.0, 100.0, 0.0]).to(dtype)
    flat = c[:, None].expand(4, cols).contiguous()
    y = O.rms_norm_ref(flat, w, eps).double()
    closed = (c.double() / torch.sqrt(c.double() ** 2 + eps))[:, None] * wd[None, :]
    assert torch.all((y - closed).abs() <= 1.01 * _step(closed, dtype) + 1e-6 * closed.abs() + 1e-30)
    assert torch.all(y[3] == 0)
    # eps = 0 and a power-of-two factor: the normalised value does not change at all
    a = O.rms_norm_ref(x, w, 0.0)
    b = O.rms_norm_ref((x.float() * 8.0).to(dtype), w, 0.0)
    assert torch.equal(a, b)
    # unit weight, eps = 0: the result has unit mean square
    ones = torch.ones(cols, dtype=dtype)
    ms = (O.rms_norm_ref(x, ones, 0.0).double() ** 2).mean(1)
    torch.testing.assert_close(ms, torch.ones_like(ms), rtol=4 * torch.finfo(dtype).eps, atol=0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_fused_add_rms_norm_ref_pinned(dtype):
    g = torch.Generator().manual_seed(4)
    rows, cols, eps = 16, 2048, 1e-6
    x = torch.randn(rows, cols, generator=g).to(dtype)
    r = (3 * torch.randn(rows, cols, generator=g)).to(dtype)
    w = (1 + 0.2 * torch.randn(cols, generator=g)).to(dtype)
    y, new_r = O.fused_add_rms_norm_ref(x, r, w, eps)
    t = x.double() + r.double()
    # the new residual is the sum rounded once
    assert torch.equal(new_r, (x.float() + r.float()).to(dtype))
    assert torch.all((new_r.double() - t).abs() <= 0.51 * _step(t, dtype) + 1e-30)
    # y from the *stored* sum, the variance from the unrounded one
    exact = new_r.double() / torch.sqrt((t * t).mean(1, keepdim=True) + eps) * w.double()
    assert torch.all((y.double() - exact).abs() <= 0.51 * _step(exact, dtype) + 4e-7 * exact.abs() + 1e-30)
    # with a zero residual and fp32 tensors the two operators differ only in where they round: same values here
    if dtype == torch.float32:
        y0, r0 = O.fused_add_rms_norm_ref(x, torch.zeros_like(x), w, eps)
        assert torch.equal(r0, x)
        torch.testing.assert_close(y0, O.rms_norm_ref(x, w, eps), rtol=3e-7, atol=1e-30)
        lib = torch.nn.functional.rms_norm(t.float(), (cols,), w, eps)
        torch.testing.assert_close(y, lib, rtol=1e-6, atol=1e-30)
