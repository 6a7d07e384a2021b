"""fp16 results at large M: the kernels that serve bf16 there write fp16 through the same stores.

The reference's own block-GEMM test asks for fp16 (tests/test_w8a8_block_fp8_matmul.py:107, atol 1e-4 * K, rtol 1e-3);
cutlass_scaled_mm takes the output type from `c` (src/flag_gems/fused/cutlass_scaled_mm.py:394-402).  Beyond the
reference's tolerance the fp16 result must be the fp32 result of the same library rounded once: the two are computed by
different kernels (other summation orders), so a small fraction of values may land on the neighbouring fp16."""
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn


def _quantized(M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    xq, xs = O.act_quant_ref(torch.randn(M, K, generator=g).bfloat16(), 128)
    wq, ws = O.per_block_cast_to_fp8_ref((0.02 * torch.randn(N, K, generator=g)).bfloat16())
    return xq, wq, xs, ws


def _one_fp16_step(got, ref32):
    """got (fp16) against the fp32 result of another kernel: at most one fp16 step apart, few values off at all"""
    want = ref32.to(torch.float16)
    diff = (got.float() - want.float()).abs()
    # one fp16 step of the value, plus what two summation orders over K differ by in fp32 (matters near zero)
    allow = want.float().abs() * 2.0 ** -10 + 1e-6 * ref32.abs().max()
    assert (diff <= allow).all(), f"max {float((diff / allow).max())} of the allowance"
    assert (got != want).float().mean().item() < 2e-2


# whole tiles | ragged tiles | few tiles with a long K (tiles shared between compute units)
@pytest.mark.parametrize("M,N,K", [(1280, 8192, 512), (1300, 8200, 640), (512, 7168, 16384)])
def test_block_gemm_fp16_above_128_rows(M, N, K):
    xq, wq, xs, ws = _quantized(M, N, K, seed=N)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=torch.float16)
    assert got.dtype == torch.float16 and got.shape == (M, N)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32)
    torch.testing.assert_close(got.cpu().float(), want, atol=1e-4 * K, rtol=1e-3)
    _one_fp16_step(got.cpu(), flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=torch.float32).cpu())
    assert torch.equal(got, flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=torch.float16))


@pytest.mark.parametrize("M,N,K", [(1280, 8192, 512), (2000, 4112, 256)])
@pytest.mark.parametrize("use_bias", [False, True])
def test_cutlass_scaled_mm_fp16_above_128_rows(M, N, K, use_bias):
    g = torch.Generator().manual_seed(M)
    a = torch.randn(M, K, generator=g).to(FP8)
    b = torch.randn(N, K, generator=g).to(FP8)
    sa = torch.rand(M, 1, generator=g) * 0.1 + 0.01
    sb = torch.rand(1, N, generator=g) * 0.1 + 0.01
    bias = torch.randn(N, generator=g).to(torch.float16) if use_bias else None
    c = torch.empty(M, N, dtype=torch.float16, device=DEV)
    flag_gems.cutlass_scaled_mm(c, a.to(DEV), b.to(DEV).t(), sa.to(DEV), sb.to(DEV), bias.to(DEV) if use_bias else None)
    want = O.scaled_mm_ref(a, b.t(), sa, sb, torch.float16, bias)
    torch.testing.assert_close(c.cpu().float(), want.float(), rtol=1e-2, atol=1e-2)
    # the same sums as the bf16 call, rounded to fp16 instead (the bias, where there is one, in the type of its call)
    c_bf = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    flag_gems.cutlass_scaled_mm(c_bf, a.to(DEV), b.to(DEV).t(), sa.to(DEV), sb.to(DEV), bias.bfloat16().to(DEV) if use_bias else None)
    mag = c_bf.float().abs().cpu() + (bias.float().abs() if use_bias else 0.0)
    assert ((c.cpu().float() - c_bf.cpu().float()).abs() <= mag * 2.0 ** -7 + 1e-6).all()
    # and finer than bf16 could be: against the fp32 result of the tile kernel, one fp16 step plus the noise of two
    # summation orders (the matrix instruction aligns the 128 products of a K-block before it adds them)
    c32 = torch.empty(M, N, dtype=torch.float32, device=DEV)
    flag_gems.cutlass_scaled_mm(c32, a.to(DEV), b.to(DEV).t(), sa.to(DEV), sb.to(DEV), None)
    if not use_bias:
        diff = (c.cpu().float() - c32.cpu()).abs()
        assert (diff <= c32.cpu().abs() * 2.0 ** -10 + 1e-3 * c32.abs().mean().item()).all()


def test_int8_cutlass_scaled_mm_fp16_above_128_rows():
    M, N, K = 1280, 4096, 512
    g = torch.Generator().manual_seed(3)
    a = torch.round((torch.randn(M, K, generator=g) * 5).clamp(-128, 127)).to(torch.int8)
    b = torch.round((torch.randn(N, K, generator=g) * 5).clamp(-128, 127)).to(torch.int8)
    sa = torch.rand(M, 1, generator=g) * 0.02 + 0.001
    sb = torch.rand(1, N, generator=g) * 0.02 + 0.001
    bias = torch.randn(N, generator=g).to(torch.float16)
    c = torch.empty(M, N, dtype=torch.float16, device=DEV)
    flag_gems.cutlass_scaled_mm(c, a.to(DEV), b.to(DEV).t(), sa.to(DEV), sb.to(DEV), bias.to(DEV))
    # exact sums, scaled in fp32 in the kernel's order, rounded once, bias added in fp16: every bit is determined
    mine = (((a.double() @ b.double().t()).float() * sa) * sb).to(torch.float16) + bias
    assert torch.equal(c.cpu(), mine)


def test_grouped_gemm_fp16():
    M, N, K, E = 700, 512, 1024, 4
    ends = torch.tensor([100, 400, 400, 700], dtype=torch.int32)
    g = torch.Generator().manual_seed(11)
    xq, xs = O.act_quant_ref(torch.randn(M, K, generator=g).bfloat16(), 128)
    wq, ws = [], []
    for _ in range(E):
        q, s = O.per_block_cast_to_fp8_ref((0.02 * torch.randn(N, K, generator=g)).bfloat16())
        wq.append(q)
        ws.append(s)
    wq, ws = torch.stack(wq), torch.stack(ws)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), ends.to(DEV), [128, 128])
    got = flag_gems.grouped_w8a8_block_fp8_matmul(*args, output_dtype=torch.float16)
    assert got.dtype == torch.float16
    want = O.grouped_block_fp8_matmul_ref(xq, wq, xs, ws, ends, [128, 128])
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    # the same sums as the bf16 call, rounded to the other type: never further from it than the two roundings allow
    bf = flag_gems.grouped_w8a8_block_fp8_matmul(*args).cpu().float()
    assert ((got.cpu().float() - bf).abs() <= bf.abs() * 2.0 ** -7 + 1e-6).all()
    # few rows per segment (short tiles, tiles cut along K)
    ends2 = torch.tensor([5, 30, 30, 64], dtype=torch.int32)
    args2 = (xq[:64].to(DEV), wq.to(DEV), xs[:64].to(DEV), ws.to(DEV), ends2.to(DEV), [128, 128])
    got2 = flag_gems.grouped_w8a8_block_fp8_matmul(*args2, output_dtype=torch.float16)
    want2 = O.grouped_block_fp8_matmul_ref(xq[:64], wq, xs[:64], ws, ends2, [128, 128])
    torch.testing.assert_close(got2.cpu().float(), want2, rtol=1e-2, atol=1e-2)
