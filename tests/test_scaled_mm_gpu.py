"""GPU parity of cutlass_scaled_mm and aten::_scaled_mm against the CPU oracle.

Shapes follow the reference's test kits (tests/test_cutlass_scaled_mm.py:65-85,
tests/test_scaled_mm.py:32-36); the bar is rtol 1e-2 / atol 1e-2, far tighter than the
reference's own (rtol 0.5, atol 0.15)."""
import os

import numpy as np
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

MNK = [
    (1, 256, 128), (1, 16384, 1024), (1, 24576, 512), (16, 256, 512), (16, 16384, 128), (16, 24576, 4096),
    (32, 8192, 4096), (32, 16384, 4096), (33, 1024, 1024), (33, 8192, 128), (64, 2048, 512), (64, 16384, 1024),
    (100, 8192, 512), (100, 1024, 4096), (48, 640, 4096), (128, 32768, 4096), (256, 4096, 4096), (512, 256, 1024), (512, 8192, 4096),
    (512, 16384, 128), (512, 24576, 128), (8, 20496, 1536),
    # 16 rows against long K: the activations pass through two LDS slots per wavefront, pair by pair
    (16, 4608, 7296), (13, 7168, 16384),
    # 17 to 32 rows against wide weights and short K: a wavefront per 16 weight rows, two 16-row images of the activations in LDS
    (24, 24576, 512), (32, 20496, 1536), (17, 32768, 256), (40, 24592, 1536), (33, 49152, 2048),
    # 17 to 32 rows against weights of up to 6144 rows: two parts of up to 16 rows on the decode kernels in one launch
    (32, 2112, 7168), (24, 4624, 7168), (30, 4096, 4096), (18, 2304, 16384),
    # 65 to 128 rows against small weights: the staged-activation kernel over the two halves of the rows
    (65, 2112, 7168), (100, 1040, 8192), (128, 4096, 4096), (77, 8192, 1024),
    # 33 to 64 rows against small weights: four parts of up to 16 rows on the decode kernels ((100, 1040, 8192) above: eight)
    (33, 512, 7168), (50, 1040, 8192), (64, 2048, 2048),
    # few 256 x 256 tiles with a long K: compute units share tiles and add their sums through the workspace
    (384, 5632, 8320), (300, 3088, 8448),
    # K that is not a multiple of 128 (operands go through registers), above and below 128 rows
    (300, 1040, 4160), (1030, 2064, 1040), (40, 528, 400),
]


def _inputs(M, N, K, seed, a_kind, b_kind):
    g = torch.Generator().manual_seed(seed)
    a = torch.clamp(torch.randn(M, K, generator=g), -448, 448).to(FP8)
    b = torch.clamp(torch.randn(K, N, generator=g), -448, 448).t().contiguous().t().to(FP8)
    sa = torch.randn((M,) if a_kind == "vector" else (1,), generator=g)
    sb = torch.randn((N,) if b_kind == "vector" else (1,), generator=g)
    return a, b, sa, sb


@pytest.mark.parametrize("M,N,K", MNK)
@pytest.mark.parametrize("kinds", [("scalar", "scalar"), ("vector", "vector"), ("vector", "scalar"), ("scalar", "vector")])
@pytest.mark.parametrize("use_bias", [False, True])
def test_cutlass_scaled_mm(M, N, K, kinds, use_bias):
    if M * N * K > 2 ** 33 and (kinds[0] != kinds[1]):
        pytest.skip("largest shapes run with the two symmetric scale kinds only (CPU oracle time)")
    a, b, sa, sb = _inputs(M, N, K, 0, *kinds)
    bias = torch.randn(N, generator=torch.Generator().manual_seed(1)).bfloat16() if use_bias else None
    want = O.scaled_mm_ref(a, b, sa, sb, torch.bfloat16, bias)
    c = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ret = flag_gems.cutlass_scaled_mm(c, a.to(DEV), b.to(DEV).t().contiguous().t(), sa.to(DEV), sb.to(DEV),
                                      bias.to(DEV) if use_bias else None)
    assert ret is None
    # rtol/atol 1e-2 against the unrounded fp32 result.  The reference rounds to bf16 twice (cast,
    # then bias add in bf16), so where product and bias cancel the allowance follows their
    # magnitudes, not the sum's; comparing two double-rounded bf16 results with each other would
    # need 2 ulp = 1.6e-2.
    prod = O.scaled_mm_ref(a, b, sa, sb, torch.float32)
    exact = prod + bias.float() if use_bias else prod
    # randn scales make outputs O(100); the absolute term is 1e-2 of the typical output magnitude
    atol = 1e-2 * max(1.0, float(prod.abs().mean()))
    allow = 1e-2 * (prod.abs() + (bias.float().abs() if use_bias else 0.0)) + atol
    err = (c.cpu().float() - exact).abs()
    assert (err <= allow).all(), f"max excess {(err - allow).max().item()}"
    assert ((want.float() - exact).abs() <= allow).all()  # the oracle's own rounding fits the same allowance


def test_bias_is_added_after_the_cast():
    a, b, sa, sb = _inputs(64, 256, 512, 2, "vector", "vector")
    bias = torch.randn(256, generator=torch.Generator().manual_seed(3)).bfloat16()
    c0 = torch.empty(64, 256, dtype=torch.bfloat16, device=DEV)
    c1 = torch.empty_like(c0)
    args = (a.to(DEV), b.to(DEV).t().contiguous().t(), sa.to(DEV), sb.to(DEV))
    flag_gems.cutlass_scaled_mm(c0, *args)
    flag_gems.cutlass_scaled_mm(c1, *args, bias.to(DEV))
    assert torch.equal(c1, c0 + bias.to(DEV))  # bf16 + bf16 -> bf16, exactly the reference's epilogue


def test_golden_vector():
    z = np.load(os.path.join(GOLD, "scaled_mm.npz"))
    a = torch.from_numpy(z["a"]).view(FP8).to(DEV)
    b = torch.from_numpy(z["b_t"]).view(FP8).to(DEV).t()
    bias = torch.from_numpy(z["bias_bits"]).view(torch.bfloat16).to(DEV)
    c = torch.empty(32, 64, dtype=torch.bfloat16, device=DEV)
    flag_gems.cutlass_scaled_mm(c, a, b, torch.from_numpy(z["sa"]).to(DEV).reshape(-1), torch.from_numpy(z["sb"]).to(DEV).reshape(-1), bias)
    want = torch.from_numpy(z["out_bits"]).view(torch.bfloat16)
    torch.testing.assert_close(c.cpu().float(), want.float(), rtol=1e-2, atol=1e-2)


def test_blockwise_branch_equals_block_gemm():
    g = torch.Generator().manual_seed(4)
    M, N, K = 40, 384, 512
    a = torch.randn(M, K, generator=g).to(FP8)
    w = torch.randn(N, K, generator=g).to(FP8)
    a_s = 0.01 * torch.rand(M, K // 128, generator=g) + 0.005
    w_s = 0.01 * torch.rand(N // 128, K // 128, generator=g) + 0.005
    want = O.block_fp8_matmul_dequant_ref(a, w, a_s, w_s, [128, 128], torch.float32)
    c = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    b = w.to(DEV).t()                       # [K, N] column-major
    b_s = w_s.to(DEV).t()                   # [K/128, N/128]
    flag_gems.cutlass_scaled_mm(c, a.to(DEV), b, a_s.to(DEV), b_s)
    torch.testing.assert_close(c.cpu().float(), want, rtol=1e-2, atol=1e-2)
    with pytest.raises(AssertionError):
        flag_gems.cutlass_scaled_mm(c, a.to(DEV), b, a_s.to(DEV), b_s, torch.zeros(N, dtype=torch.bfloat16, device=DEV))


def test_assertions_and_unsupported():
    a, b, sa, sb = (t.to(DEV) for t in _inputs(16, 256, 128, 5, "vector", "vector"))
    b = b.t().contiguous().t()
    c = torch.empty(16, 256, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(AssertionError):
        flag_gems.cutlass_scaled_mm(c, a, b.contiguous(), sa, sb)          # b row-major
    with pytest.raises(AssertionError):
        flag_gems.cutlass_scaled_mm(c[:, :128], a, b, sa, sb)              # shape mismatch
    with pytest.raises(AssertionError):
        flag_gems.cutlass_scaled_mm(c, a, b, sa.double(), sb)              # scale dtype
    with pytest.raises(AssertionError):
        flag_gems.cutlass_scaled_mm(c, a, b, sa, sb, torch.zeros(3, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(NotImplementedError):  # int8 operands with an fp8 output
        ai = torch.ones(16, 128, dtype=torch.int8, device=DEV)
        bi = torch.ones(256, 128, dtype=torch.int8, device=DEV).t()
        flag_gems.cutlass_scaled_mm(torch.empty(16, 256, dtype=FP8, device=DEV), ai, bi, sa, sb)


# ----------------------------------------------------------------- aten::_scaled_mm
def _make_scales(rows, cols, mode):
    if mode == "scalar":
        return torch.tensor([0.75]), torch.tensor([1.25])
    sa = torch.linspace(0.75, 1.25, rows)
    sb = torch.linspace(1.25, 0.75, cols)
    if mode == "rowwise_2d":
        return sa.reshape(rows, 1), sb.reshape(1, cols)
    return sa, sb


@pytest.mark.parametrize("M,N,K", [(16, 16, 16), (17, 31, 32), (64, 48, 80), (256, 512, 1024)])
@pytest.mark.parametrize("case", [(None, "scalar", False), (torch.float16, "rowwise_1d", True),
                                  (torch.float32, "rowwise_2d", True), (torch.bfloat16, "rowwise_2d", False)])
def test_aten_scaled_mm_under_use_gems(M, N, K, case):
    out_dtype, scale_mode, use_bias = case
    g = torch.Generator().manual_seed(0)
    mat1 = (torch.randn(M, K, generator=g) * 0.25).to(FP8)
    mat2 = (torch.randn(K, N, generator=g) * 0.25).to(FP8)    # row-major, as the reference test passes it
    sa, sb = _make_scales(M, N, scale_mode)
    bias = None
    if use_bias:
        bias = (torch.randn(N, generator=g) * 0.25).to(out_dtype or torch.float32)
    ref = O.scaled_mm_ref_postscale(mat1, mat2, sa, sb, bias, out_dtype)
    mat2_dev = mat2.to(DEV)
    if K % 16 == 0 and N % 16 == 0:
        mat2_dev = mat2_dev.t().contiguous().t()   # what native torch._scaled_mm requires
    with flag_gems.use_gems():
        assert "_scaled_mm" in flag_gems.all_registered_keys()
        res = torch._scaled_mm(mat1.to(DEV), mat2_dev, sa.to(DEV), sb.to(DEV),
                               bias=bias.to(DEV) if use_bias else None,
                               scale_result=torch.tensor([2.0], device=DEV), out_dtype=out_dtype, use_fast_accum=True)
    assert res.dtype == (out_dtype or FP8) and res.shape == (M, N)
    if out_dtype is None:
        # fp8 output: one e4m3 rounding step (2^-3 relative) at most
        torch.testing.assert_close(res.float().cpu(), ref.float(), atol=0.125, rtol=0.5)
        torch.testing.assert_close(res.float().cpu(), ref.float(), atol=2 ** -7, rtol=2 ** -3)
    else:
        torch.testing.assert_close(res.float().cpu(), ref.float(), rtol=1e-2, atol=1e-2)


def test_aten_scaled_mm_out_returns_out():
    g = torch.Generator().manual_seed(1)
    mat1 = (torch.randn(16, 32, generator=g) * 0.25).to(FP8).to(DEV)
    mat2 = (torch.randn(32, 16, generator=g) * 0.25).to(FP8).to(DEV).t().contiguous().t()
    sa, sb = (t.to(DEV) for t in _make_scales(16, 16, "rowwise_2d"))
    bias = (torch.randn(1, 16, generator=g) * 0.25).to(DEV)
    out = torch.empty(16, 16, dtype=torch.float32, device=DEV)
    with flag_gems.use_gems():
        ret = torch.ops.aten._scaled_mm.out(mat1, mat2, sa, sb, bias=bias, scale_result=None,
                                            out_dtype=torch.float32, use_fast_accum=False, out=out)
    assert ret is out
    ref = O.scaled_mm_ref_postscale(mat1.cpu(), mat2.cpu(), sa.cpu(), sb.cpu(), bias.cpu(), torch.float32)
    torch.testing.assert_close(out.cpu(), ref, rtol=2e-3, atol=2e-4)


def test_scaled_mm_errors():
    a = torch.zeros(4, 16, dtype=FP8, device=DEV)
    b = torch.zeros(16, 8, dtype=FP8, device=DEV).t().contiguous().t()
    one = torch.ones(1, device=DEV)
    with pytest.raises(RuntimeError):
        flag_gems.scaled_mm(a, b[:8], one, one)
    with pytest.raises(RuntimeError):
        flag_gems.scaled_mm(a, b, torch.ones(3, device=DEV), one)
    with pytest.raises(RuntimeError):
        flag_gems.scaled_mm(a, b, one, one, bias=torch.ones(5, device=DEV))
    with pytest.raises(RuntimeError):
        flag_gems.scaled_mm_out(a, b, one, one, out_dtype=torch.float16, out=torch.empty(4, 8, device=DEV))
    out = flag_gems.scaled_mm(a[:0], b, one, one, out_dtype=torch.bfloat16)
    assert out.shape == (0, 8)


def test_vllm_cutlass_scaled_mm_op():
    flag_gems.patch_empty_vllm()
    a, b, sa, sb = (t.to(DEV) for t in _inputs(33, 256, 512, 6, "vector", "vector"))
    b = b.t().contiguous().t()
    c = torch.empty(33, 256, dtype=torch.float16, device=DEV)
    torch.ops._C.cutlass_scaled_mm(c, a, b, sa, sb, None)
    want = O.scaled_mm_ref(a.cpu(), b.cpu(), sa.cpu(), sb.cpu(), torch.float16)
    torch.testing.assert_close(c.cpu().float(), want.float(), rtol=1e-2, atol=1e-2)
