"""Block-scaled FP8 GEMM with power-of-two scales: the path that hands the scales to the matrix instruction as E8M0
exponents (fg_block_fp8_gemm_pow2_scales), against the CPU oracle and against the fp32-scale path on the same inputs.

Tolerance: rtol/atol 1e-2 for the bf16 result against the float64 dequantised matmul (the bar of every block GEMM
test, reference tests/test_w8a8_block_fp8_matmul.py:76-100 restated), and at most one bf16 step between the two device
paths: a power-of-two scale is exact in both, only the order of the fp32 roundings differs."""
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn


def _pow2_inputs(M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(M, K, generator=g) * torch.logspace(-2, 1, M).unsqueeze(1)).bfloat16()
    w = (0.02 * torch.randn(N, K, generator=g)).bfloat16()
    xq, xs = O.act_quant_ref(x, 128, "ue8m0")
    wq, ws = O.per_block_cast_to_fp8_ref(w, use_ue8m0=True)
    for s in (xs, ws):
        m, _ = torch.frexp(s)
        assert torch.all(m == 0.5)  # powers of two
    return xq, wq, xs, ws


# persistent kernel: whole tiles (aligned and with edges), several rounds, stream-K, equal cuts, the two-launch tail
SHAPES = [(512, 24576, 1536), (1100, 13400, 384), (4096, 2112, 7168), (2048, 2112, 7168), (512, 7168, 16384),
          (2304, 8192, 2048), (300, 10000, 1024), (4096, 4608, 1024)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_pow2_scales_match_the_oracle_and_the_fp32_scale_path(M, N, K):
    xq, wq, xs, ws = _pow2_inputs(M, N, K, seed=M + N)
    a, b, a_s, b_s = xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV)
    plain = flag_gems.w8a8_block_fp8_matmul(a, b, a_s, b_s, [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(a, b, a_s, b_s, [128, 128], scales_are_powers_of_two=True)
    assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    # sampled rows x sampled 128-column blocks against the float64 oracle (a full product would take minutes)
    rows = sorted({0, 1, 63, 64, 255, 256, M // 2, M - 2, M - 1} & set(range(M)))
    nb = (N + 127) // 128
    cols = torch.cat([torch.arange(c * 128, min((c + 1) * 128, N)) for c in sorted({0, 1 % nb, nb // 2, nb - 1})])
    r = torch.tensor(rows)
    want = O.block_fp8_matmul_dequant_ref(xq[r], wq[cols], xs[r], ws[torch.unique(cols // 128)], [128, 128],
                                          torch.float32, torch.float64)
    sub = got[r.to(DEV)][:, cols.to(DEV)].cpu().float()
    torch.testing.assert_close(sub, want, rtol=1e-2, atol=1e-2)
    # one bf16 step at most between the two paths, everywhere
    diff = (got.float() - plain.float()).abs()
    step = plain.float().abs() * 2.0 ** -7 + 1e-30
    assert float((diff / step).max()) <= 1.0 + 1e-6, f"max difference {float((diff / step).max())} bf16 steps"
    again = flag_gems.w8a8_block_fp8_matmul(a, b, a_s, b_s, [128, 128], scales_are_powers_of_two=True)
    assert torch.equal(again.view(torch.int16), got.view(torch.int16))


def test_e8m0_scale_tensors_take_the_same_path():
    """fp8_matmul(scale_dtype=float8_e8m0fnu) (reference src/flag_gems/ops/fp8_matmul.py:165-167) and
    w8a8_block_fp8_matmul with E8M0 scale tensors give the bits of the call that was promised powers of two."""
    M, N, K = 640, 4096, 2048
    xq, wq, xs, ws = _pow2_inputs(M, N, K, seed=5)
    a, b, a_s, b_s = xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV)
    a8, b8 = a_s.to(torch.float8_e8m0fnu), b_s.to(torch.float8_e8m0fnu)
    assert torch.equal(a8.float(), a_s) and torch.equal(b8.float(), b_s)
    promised = flag_gems.w8a8_block_fp8_matmul(a, b, a_s, b_s, [128, 128], scales_are_powers_of_two=True)
    assert torch.equal(flag_gems.fp8_matmul(a, a8, b, b8, scale_dtype=torch.float8_e8m0fnu).view(torch.int16), promised.view(torch.int16))
    assert torch.equal(flag_gems.w8a8_block_fp8_matmul(a, b, a8, b8, [128, 128]).view(torch.int16), promised.view(torch.int16))


def test_small_problems_run_the_usual_kernels():
    """Where the persistent kernel does not take the problem the promise changes nothing: the same bits."""
    for (M, N, K) in [(8, 2112, 7168), (64, 4096, 512), (128, 1300, 4096), (300, 520, 200)]:
        xq, wq, xs, ws = _pow2_inputs(M, N, (K + 127) // 128 * 128, seed=M)
        if K % 128:
            xq, wq = xq[:, :K].contiguous(), wq[:, :K].contiguous()
        a, b, a_s, b_s = xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV)
        plain = flag_gems.w8a8_block_fp8_matmul(a, b, a_s, b_s, [128, 128])
        got = flag_gems.w8a8_block_fp8_matmul(a, b, a_s, b_s, [128, 128], scales_are_powers_of_two=True)
        assert torch.equal(got.view(torch.int16), plain.view(torch.int16)), (M, N, K)
