"""The benchmark configurations at their full sizes, through the HIP path, against the CPU oracle.

The shapes are the ones the benchmark driver times (Llama-3-8B linears, DeepSeek-V3 GEMMs, the 8192-square
per-token x per-channel scaled GEMM, Mixtral expert layers): the launch planner picks its kernel variant from
(M, N, K), so these exact shapes must run under a checker, not only look-alikes.  A full-size matmul on the host
would take minutes, so the oracle is evaluated on a sample: a handful of activation rows (first, last, rows next to
tile boundaries; for expert layers the first and last row of every segment) times whole 128-column scale blocks of
the weight (first, second, one in the middle, the last, which may be ragged).  Every output element is a dot product
of one activation row and one weight row, so any indexing mistake that moves rows, columns, K-blocks or scales
shows in such a sample; on top, a second call must give the same bits, and the whole result is compared on the
device with torch's own fp32 GEMM of the dequantised operands (an independent implementation that sees every tile,
K cut and tail launch the planner issues for the shape).

Tolerance: |got - want| <= 1e-2 + 1e-2 |want| for the bf16 result against the float64 dequantised matmul
(reference tests/test_w8a8_block_fp8_matmul.py:76-100 restated; the reference's own bar is looser)."""
import functools

import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn


@functools.lru_cache(maxsize=16)
def _weight(N, K, seed=0):
    """W ~ N(0, 0.02) bf16 quantized per 128 x 128 block on the device (the device quantizer is bit-exact with the
    oracle's, tests/test_block_quant_gpu.py)."""
    g = torch.Generator(device=DEV).manual_seed(seed + N * 7 + K)
    w = (0.02 * torch.randn(N, K, device=DEV, generator=g)).bfloat16()
    return flag_gems.per_block_cast_to_fp8(w)


def _activation(M, K, seed=0):
    g = torch.Generator(device=DEV).manual_seed(seed + M * 13 + K)
    x = torch.randn(M, K, device=DEV, generator=g).bfloat16()
    return flag_gems.act_quant_triton(x, 128)


def _sample_rows(M):
    cand = [0, 1, 15, 16, 63, 64, 127, 128, 255, 256, 257, M // 2, M - 2, M - 1]
    return sorted({r for r in cand if 0 <= r < M})[:12]


def _sample_blocks(N):
    nb = (N + 127) // 128
    return sorted({0, 1 % nb, nb // 2, nb - 2 if nb > 1 else 0, nb - 1})  # the last one may be ragged: it stays last


def _oracle_on_sample(xq, wq, xs, ws, rows, blocks):
    N = wq.shape[0]
    cols = torch.cat([torch.arange(b * 128, min((b + 1) * 128, N)) for b in blocks])
    r = torch.tensor(rows)
    a = xq.view(torch.uint8)[r.to(xq.device)].cpu().view(FP8)
    b = wq.view(torch.uint8)[cols.to(wq.device)].cpu().view(FP8)
    want = O.block_fp8_matmul_dequant_ref(a, b, xs[r.to(xs.device)].cpu(), ws[torch.tensor(blocks).to(ws.device)].cpu(),
                                          [128, 128], torch.float32, torch.float64)
    return r, cols, want


def _dequantized_weight(wq, ws):
    """fp32 W[n, k] * Ws[n // 128, k // 128] on the device."""
    N, K = wq.shape
    s = ws.repeat_interleave(128, dim=0)[:N].repeat_interleave(128, dim=1)[:, :K]
    return wq.float() * s


def _assert_whole_matrix(got, xq, xs, w_deq, what=""):
    """Every element of `got` against torch's own fp32 GEMM of the dequantised operands, computed on the device in
    row chunks.  This is a cross-check, not the oracle: torch.matmul shares no code with libflaggems_amd.so, and
    unlike the sampled oracle comparison it sees every tile, every K cut and every tail launch of the call."""
    M, K = xq.shape
    bad, worst, where = 0, 0.0, None
    for r0 in range(0, M, 1024):
        r1 = min(M, r0 + 1024)
        x_deq = xq[r0:r1].float() * xs[r0:r1].repeat_interleave(128, dim=1)[:, :K]
        ref = x_deq @ w_deq.t()
        excess = (got[r0:r1].float() - ref).abs() - (1e-2 + 1e-2 * ref.abs())
        n_bad = int((excess > 0).sum())
        if n_bad:
            bad += n_bad
            top = float(excess.max())
            if top > worst:
                idx = int(excess.argmax())
                worst, where = top, (r0 + idx // ref.shape[1], idx % ref.shape[1])
    assert bad == 0, f"{what}: {bad} of {got.numel()} elements outside rtol/atol 1e-2 of the fp32 product, worst excess {worst:.3g} at {where}"


def _check_block_gemm(M, N, K):
    xq, xs = _activation(M, K)
    wq, ws = _weight(N, K)
    got = flag_gems.w8a8_block_fp8_matmul(xq, wq, xs, ws, [128, 128])
    assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    r, cols, want = _oracle_on_sample(xq, wq, xs, ws, _sample_rows(M), _sample_blocks(N))
    sub = got[r.to(DEV)][:, cols.to(DEV)].cpu().float()
    torch.testing.assert_close(sub, want, rtol=1e-2, atol=1e-2)
    # at most one bf16 rounding plus fp32 accumulation noise
    err = (sub.double() - want.double()).abs()
    assert float((err / (want.double().abs() / 128 + 2e-3)).max()) < 1.0
    again = flag_gems.w8a8_block_fp8_matmul(xq, wq, xs, ws, [128, 128])
    assert torch.equal(again.view(torch.int16), got.view(torch.int16)), "two runs of one problem differ"
    assert torch.isfinite(got.float()).all()
    _assert_whole_matrix(got, xq, xs, _dequantized_weight(wq, ws), f"M={M} N={N} K={K}")


LLAMA3_8B = [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]
DSV3 = [(2112, 7168), (24576, 1536), (32768, 512), (7168, 16384), (4608, 7168), (7168, 2304)]


@pytest.mark.parametrize("N,K", LLAMA3_8B)
@pytest.mark.parametrize("M", [1, 16, 128, 1024, 4096])
def test_llama3_8b_linears(M, N, K):
    _check_block_gemm(M, N, K)


@pytest.mark.parametrize("N,K", DSV3)
@pytest.mark.parametrize("M", [1, 8, 16, 64, 512, 2048, 4096])
def test_deepseek_v3_gemms(M, N, K):
    _check_block_gemm(M, N, K)


@pytest.mark.parametrize("use_bias", [False, True])
@pytest.mark.parametrize("M", [1, 32, 256, 2048, 8192])
def test_cutlass_scaled_mm_8192_square(M, use_bias):
    """Per-token x per-channel scaled GEMM of the reference benchmark (benchmark/test_cutlass_scaled_mm.py:70-91):
    N = K = 8192, sources ~ N(0, 1), scales amax / 448 per row of A and per column of B, B column-major, bf16 out,
    optional bf16 bias added after the cast (tests/test_cutlass_scaled_mm.py:154-187 restated by the oracle)."""
    N = K = 8192
    g = torch.Generator(device=DEV).manual_seed(M)
    a32 = torch.randn(M, K, device=DEV, generator=g)
    b32 = torch.randn(K, N, device=DEV, generator=g)
    sa = a32.abs().amax(dim=1, keepdim=True) / 448.0        # [M, 1]
    sb = b32.abs().amax(dim=0, keepdim=True) / 448.0        # [1, N]
    a = (a32 / sa).to(FP8)
    b = (b32 / sb).t().contiguous().to(FP8).t()             # [K, N] with stride(0) == 1
    assert b.stride(0) == 1
    bias = torch.randn(N, device=DEV, generator=g).bfloat16() if use_bias else None
    c = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    assert flag_gems.cutlass_scaled_mm(c, a, b, sa, sb, bias) is None
    rows = torch.tensor(_sample_rows(M))
    a_rows = a.view(torch.uint8)[rows.to(DEV)].cpu().view(FP8)
    b_cpu = b.view(torch.uint8).cpu().view(FP8)
    prod = O.scaled_mm_ref(a_rows, b_cpu, sa[rows.to(DEV)].cpu(), sb.cpu(), torch.float32)
    exact = prod + bias.cpu().float() if use_bias else prod
    # the reference rounds to bf16 twice when there is a bias (cast, then the add in bf16): where product and bias
    # cancel, the allowance follows their magnitudes, not the sum's
    allow = 1e-2 * (prod.abs() + (bias.cpu().float().abs() if use_bias else 0.0)) + 1e-2
    err = (c[rows.to(DEV)].cpu().float() - exact).abs()
    assert (err <= allow).all(), f"max excess {(err - allow).max().item()}"
    want = O.scaled_mm_ref(a_rows, b_cpu, sa[rows.to(DEV)].cpu(), sb.cpu(), torch.bfloat16, bias.cpu() if use_bias else None)
    assert ((want.float() - exact).abs() <= allow).all()
    c2 = torch.empty_like(c)
    flag_gems.cutlass_scaled_mm(c2, a, b, sa, sb, bias)
    assert torch.equal(c2.view(torch.int16), c.view(torch.int16))
    # every element against torch's fp32 GEMM of the scaled operands, on the device in row chunks (a cross-check
    # that sees every tile of the launch; the allowance is the one of the sampled oracle comparison above)
    b_deq = b.float() * sb
    for r0 in range(0, M, 1024):
        r1 = min(M, r0 + 1024)
        prod_d = (a[r0:r1].float() * sa[r0:r1]) @ b_deq
        exact_d = prod_d + bias.float() if use_bias else prod_d
        allow_d = 1e-2 * (prod_d.abs() + (bias.float().abs() if use_bias else 0.0)) + 1e-2
        err_d = (c[r0:r1].float() - exact_d).abs()
        assert bool((err_d <= allow_d).all()), f"rows {r0}..{r1}: max excess {(err_d - allow_d).max().item()}"


@functools.lru_cache(maxsize=2)
def _expert_weights(N, K):
    qs, ss = [], []
    for e in range(8):
        g = torch.Generator(device=DEV).manual_seed(1000 + e + N)
        q, s = flag_gems.per_block_cast_to_fp8((0.02 * torch.randn(N, K, device=DEV, generator=g)).bfloat16())
        qs.append(q)
        ss.append(s)
    return torch.stack(qs), torch.stack(ss)


@pytest.mark.parametrize("N,K", [(28672, 4096), (4096, 14336)])
@pytest.mark.parametrize("T", [64, 1024, 4096])
def test_mixtral_expert_layers(T, N, K):
    """8 experts, top-2 routing of T tokens with Zipf(1.1)-skewed loads, rows sorted by expert: W1 [8, 28672, 4096]
    and W2 [8, 4096, 14336].  Oracle: the per-expert loop of tests/test_fused_experts_impl.py:604-662 on the first,
    second and last row of every expert's segment."""
    ends = O.make_moe_rows(T, 8, 2, seed=T)
    M = 2 * T
    assert int(ends[-1]) == M
    xq, xs = _activation(M, K, seed=5)
    wq, ws = _expert_weights(N, K)
    got = flag_gems.grouped_w8a8_block_fp8_matmul(xq, wq, xs, ws, ends.to(DEV), [128, 128])
    assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    blocks = _sample_blocks(N)
    begin = 0
    checked = 0
    for e in range(8):
        end = int(ends[e])
        if end > begin:
            rows = sorted({begin, min(begin + 1, end - 1), (begin + end) // 2, end - 1})
            r, cols, want = _oracle_on_sample(xq, wq[e], xs, ws[e], rows, blocks)
            sub = got[r.to(DEV)][:, cols.to(DEV)].cpu().float()
            torch.testing.assert_close(sub, want, rtol=1e-2, atol=1e-2, msg=lambda m: f"expert {e}: {m}")
            checked += len(rows)
        begin = end
    assert checked >= 8
    begin = 0
    for e in range(8):  # every row of every expert's segment against torch's fp32 GEMM on the device
        end = int(ends[e])
        if end > begin:
            _assert_whole_matrix(got[begin:end], xq[begin:end], xs[begin:end], _dequantized_weight(wq[e], ws[e]), f"expert {e}")
        begin = end
    again = flag_gems.grouped_w8a8_block_fp8_matmul(xq, wq, xs, ws, ends.to(DEV), [128, 128])
    assert torch.equal(again.view(torch.int16), got.view(torch.int16))
