"""GPU parity of the int8 branch of cutlass_scaled_mm / aten::_scaled_mm against the CPU oracle.

int8 x int8 sums are exact in int32, so the only rounding is float(sum) * scale_a * scale_b -> out dtype
(-> + bias): the result must match the oracle to one step of the output type (the reference's own tolerance for
int8 is rtol 1e-1, atol 1.0, tests/test_cutlass_scaled_mm.py:237-238).  Inputs as the reference builds them
(:48-49, :205-212): round(clamp(randn * 5, -128, 127))."""
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _to_int8(t):
    return torch.round(t.clamp(min=-128, max=127)).to(torch.int8)


def _inputs(M, N, K, seed, a_kind, b_kind):
    g = torch.Generator().manual_seed(seed)
    a = _to_int8(torch.randn(M, K, generator=g) * 5)
    b = _to_int8(torch.randn(N, K, generator=g) * 5).t()  # [K, N] column-major
    sa = torch.rand((M,) if a_kind == "vector" else (1,), generator=g) * 0.02 + 0.001
    sb = torch.rand((N,) if b_kind == "vector" else (1,), generator=g) * 0.02 + 0.001
    return a, b, sa, sb


def _exact(a, b, sa, sb):
    """int32-exact sums (float64 holds them exactly), scaled in fp32 in the kernel's order."""
    acc = (a.double() @ b.double()).float()
    sa2 = sa.reshape(-1, 1) if sa.numel() > 1 else sa.reshape(1, 1)
    sb2 = sb.reshape(1, -1) if sb.numel() > 1 else sb.reshape(1, 1)
    return acc * sa2 * sb2


@pytest.mark.parametrize("M,N,K", [(1, 256, 128), (16, 512, 512), (33, 1024, 1024), (100, 640, 4096), (256, 4096, 4096),
                                   (512, 8192, 1024), (1100, 1300, 2048), (64, 200, 192), (7, 24, 40), (1024, 2304, 512),
                                   (129, 264, 128), (700, 8, 384),
                                   # up to 32 rows: the weight-streaming kernels (K split over blocks for the first)
                                   (1, 4096, 4096), (8, 2112, 7168), (16, 7168, 2304), (32, 1024, 8192), (5, 24592, 384),
                                   (12, 32768, 512), (20, 520, 1024), (24, 32768, 512), (32, 24580, 1536),
                                   (32, 2112, 7168), (24, 4624, 7168), (16, 2304, 16384),
                                   # 65..128 rows against small weights: two halves of the rows in one launch
                                   (65, 2112, 7168), (128, 1024, 8192), (99, 4096, 4096),
                                   (47, 512, 7168), (64, 1024, 8192), (25, 6144, 4096),
                                   # 33..64 rows: the kernel with the activations of a K range in LDS
                                   (33, 2112, 7168), (64, 4096, 4096), (48, 24576, 1536), (40, 264, 512),
                                   # K that is not a multiple of 128 above 128 rows
                                   (300, 1040, 4160), (1030, 528, 1040)])
@pytest.mark.parametrize("kinds", [("scalar", "scalar"), ("vector", "vector"), ("vector", "scalar")])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16])
def test_int8_cutlass_scaled_mm(M, N, K, kinds, out_dtype):
    a, b, sa, sb = _inputs(M, N, K, 0, *kinds)
    for use_bias in (False, True):
        bias = torch.randn(N, generator=torch.Generator().manual_seed(1)).to(out_dtype) if use_bias else None
        want = O.scaled_mm_ref(a, b, sa, sb, out_dtype, bias)
        c = torch.empty(M, -(-N // 16) * 16, dtype=out_dtype, device=DEV)[:, :N]  # the reference asserts these strides
        ld = -(-K // 16) * 16
        b_dev = torch.zeros(N, ld, dtype=torch.int8, device=DEV)
        b_dev[:, :K] = b.t().to(DEV)
        flag_gems.cutlass_scaled_mm(c, a.to(DEV), b_dev[:, :K].t(), sa.to(DEV), sb.to(DEV), bias.to(DEV) if use_bias else None)
        # the reference's tolerance
        torch.testing.assert_close(c.cpu(), want, rtol=1e-1, atol=1.0)
        # this build's: the exact sums, scaled in fp32, rounded once (then the bias added in the output type)
        mine = _exact(a, b, sa, sb).to(out_dtype)
        if use_bias:
            mine = mine + bias
        eps = torch.finfo(out_dtype).eps
        err = (c.cpu().double() - mine.double()).abs()
        assert torch.all(err <= mine.double().abs() * eps + 1e-6), f"max err {err.max().item()}"
        assert (c.cpu() != mine).float().mean().item() < 2e-3


def test_int8_sums_are_exact():
    """Unit scales and fp32 output: every int32 sum comes back exactly, also at the extremes of int8."""
    M, N, K = 130, 260, 1024
    g = torch.Generator().manual_seed(3)
    a = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
    b = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    a[0, :] = -128
    b[0, :] = -128
    a[1, :] = 127
    b[1, :] = -128
    one = torch.ones(1)
    c = torch.empty(M, 272, dtype=torch.float32, device=DEV)[:, :N]
    flag_gems.cutlass_scaled_mm(c, a.to(DEV), b.to(DEV).t(), one.to(DEV), one.to(DEV), None)
    want = a.double() @ b.double().t()
    assert want.abs().max() <= 2 ** 24  # exactly representable in fp32
    assert torch.equal(c.cpu().double(), want)
    assert c[0, 0].item() == 128 * 128 * K and c[1, 0].item() == -127 * 128 * K


def test_int8_sums_are_exact_in_bf16_above_128_rows():
    """bf16 output and M > 128 (the kernel that serves the large fp8 problems): sums that bf16 holds exactly come back
    exactly, on tiles inside the matrix and on ragged ones, and so do the extremes of int8."""
    g = torch.Generator().manual_seed(5)
    one = torch.ones(1, device=DEV)
    for (M, N, K) in ((512, 768, 256), (300, 520, 256), (257, 8, 128)):
        a = torch.randint(-1, 2, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
        b = torch.randint(-1, 2, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
        c = torch.empty(M, -(-N // 16) * 16, dtype=torch.bfloat16, device=DEV)[:, :N]
        flag_gems.cutlass_scaled_mm(c, a.to(DEV), b.to(DEV).t(), one, one, None)
        want = a.double() @ b.double().t()
        assert want.abs().max() <= 256
        assert torch.equal(c.cpu().double(), want), (M, N, K)
    M, N, K = 256, 256, 4096
    a = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
    b = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    a[0, :] = -128
    a[1, :] = 127
    b[0, :] = -128
    b[1, :] = 64
    c = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    flag_gems.cutlass_scaled_mm(c, a.to(DEV), b.to(DEV).t(), one, one, None)
    assert c[0, 0].item() == 128 * 128 * K and c[1, 0].item() == -127 * 128 * K  # 2^26 and -127 * 2^19
    assert c[0, 1].item() == -128 * 64 * K and c[1, 1].item() == 127 * 64 * K
    want = (a.double() @ b.double().t()).float().to(torch.bfloat16)  # one rounding of the exact sum
    assert torch.equal(c.cpu(), want)


@pytest.mark.parametrize("M,N,K", [(1, 512, 8192), (4, 2112, 7168), (16, 4096, 4096), (9, 24576, 1536), (32, 768, 2048),
                                   (33, 512, 8192), (64, 2112, 7168), (64, 4608, 7168), (16, 4608, 7168), (32, 2112, 7168), (16, 2304, 16384),
                                   (24, 2304, 16384)])
def test_int8_sums_are_exact_up_to_64_rows(M, N, K):
    """The kernels for few rows split K over wavefronts and blocks: the int32 partial sums are added as integers, so
    the fp32 result is the one rounding of the exact sum, also where the sum needs more than 24 bits."""
    g = torch.Generator().manual_seed(7)
    a = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
    b = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    a[0, :] = -128
    b[0, :] = -128
    b[1, :] = 127
    b[2, :] = (torch.arange(K) % 2 * 2 - 1).to(torch.int8) * 127  # sums that cancel
    one = torch.ones(1, device=DEV)
    c = torch.empty(M, N, dtype=torch.float32, device=DEV)
    flag_gems.cutlass_scaled_mm(c, a.to(DEV), b.to(DEV).t(), one, one, None)
    want = (a.double() @ b.double().t())
    assert want.abs().max() > 2 ** 24
    assert torch.equal(c.cpu(), want.float())
    assert c[0, 0].item() == 128 * 128 * K and c[0, 1].item() == -128 * 127 * K
    # through the C ABI: a missing workspace is refused where the kernels for few rows need one
    from flaggems_amd import _lib
    lib = _lib.load()
    a_d, b_d = a.to(DEV), b.to(DEV)
    c2 = torch.empty_like(c)
    need = lib.fg_scaled_int8_gemm_workspace_bytes(M, N, K)
    ws = _lib.workspace(torch.device(DEV), need) if need else None

    def call(ws_ptr, ws_bytes):
        return lib.fg_scaled_int8_gemm(
            a_d.data_ptr(), K, b_d.data_ptr(), K, one.data_ptr(), 0, one.data_ptr(), 0, None, _lib.FG_BF16,
            c2.data_ptr(), N, _lib.DTYPE_CODE[torch.float32], M, N, K, ws_ptr, ws_bytes,
            _lib.current_stream_ptr(torch.device(DEV)))

    _lib.check(call(ws.data_ptr() if need else None, ws.numel() if need else 0), "fg_scaled_int8_gemm")
    torch.cuda.synchronize()
    assert torch.equal(c2, c)
    if need:
        # without the workspace the call is refused, or served by a kernel that needs none (parts of up to 16 rows on the decode
        # kernels in one K range), with the same exact sums
        c2.zero_()
        rc = call(None, 0)
        assert rc in (0, -3)  # FG_ERR_WORKSPACE
        if (M, N, K) in ((64, 4608, 7168), (16, 2304, 16384)):
            assert rc == -3  # seven K ranges on the kernel of 33..64 rows (too large for the parts); two K ranges on the decode kernel
        if rc == 0:
            torch.cuda.synchronize()
            assert torch.equal(c2, c)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_int8_tiles_shared_between_compute_units_are_exact(out_dtype):
    """Few 256 x 256 tiles with a long K: compute units take ranges of K-blocks and add their int32 sums through the
    workspace.  Sparse operands keep every sum small enough for the 16-bit result to hold it exactly; the bias is
    added in the result type."""
    M, N, K = 384, 5632, 8320
    g = torch.Generator().manual_seed(9)
    a = (torch.randint(-1, 2, (M, K), generator=g) * (torch.rand(M, K, generator=g) < 0.1)).to(torch.int8)
    b = (torch.randint(-1, 2, (N, K), generator=g) * (torch.rand(N, K, generator=g) < 0.1)).to(torch.int8)
    a[0, :] = 1
    b[0, :256] = 1
    b[0, 256:] = 0
    one = torch.ones(1, device=DEV)
    bias = torch.randint(-8, 9, (N,), generator=g).to(out_dtype)
    want = a.float() @ b.float().t()  # integers far below 2^24: exact
    assert want.abs().max() <= 256 and want[0, 0] == 256
    for use_bias in (False, True):
        c = torch.empty(M, N, dtype=out_dtype, device=DEV)
        flag_gems.cutlass_scaled_mm(c, a.to(DEV), b.to(DEV).t(), one, one, bias.to(DEV) if use_bias else None)
        assert torch.equal(c.cpu().float(), want + (bias.float() if use_bias else 0.0))


def test_int8_through_aten_scaled_mm():
    a, b, sa, sb = _inputs(64, 128, 256, 4, "vector", "vector")
    want = O.scaled_mm_ref(a, b, sa, sb, torch.bfloat16)
    got = flag_gems.scaled_mm(a.to(DEV), b.to(DEV), sa.view(-1, 1).to(DEV), sb.view(1, -1).to(DEV), out_dtype=torch.bfloat16)
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=2.0 ** -7, atol=1e-3)
    with pytest.raises(NotImplementedError):
        flag_gems.scaled_mm(a.to(DEV), b.to(DEV), sa.view(-1, 1).to(DEV), sb.view(1, -1).to(DEV))  # int8 output
