"""GPU parity of w8a8_block_fp8_bmm / fp8_einsum("bhr,hdr->bhd") against the CPU oracle.

Shapes and input construction follow the reference's test (tests/test_fp8_einsum.py:46-60, 105-127).  The
reference's tolerance (rtol 2e-1, atol max(5e-2, 5 % of the largest value), :198-200) is applied, and next to it
this build's bar for the GEMM (rtol 1e-2, atol 1e-2 relative to the magnitude of the sums)."""
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O
from tests._util import assert_codes_equal, assert_scales_equal

pytestmark = pytest.mark.gpu
DEV = "cuda"

HRD = {"flash": (8, 4096, 1024), "pro": (16, 7168, 1024)}


@pytest.mark.parametrize("group", ["flash", "pro"])
@pytest.mark.parametrize("b", [1, 4, 8, 16, 32, 64, 128])
def test_einsum_reference_shapes(group, b):
    h, r, d = HRD[group]
    xq, xs, yq, ys = O.make_fp8_einsum_inputs(b, h, r, d, seed=0)
    want = O.fp8_block_einsum_ref(xq, xs, yq, ys, [128, 128])
    got = flag_gems.fp8_einsum("bhr,hdr->bhd", xq.to(DEV), xs.to(DEV), yq.to(DEV), ys.to(DEV), [128, 128])
    assert got.shape == (b, h, d) and got.dtype == torch.bfloat16 and got.is_contiguous()
    top = want.abs().max().item()
    torch.testing.assert_close(got.cpu(), want.to(torch.bfloat16), rtol=2e-1, atol=max(5e-2, top * 5e-2))
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2 * max(1.0, top / 8))


def test_einsum_large_batch_and_per_head_bits():
    """b = 4096 rows per head take the persistent kernel; every head's slice carries the bits of the plain GEMM on
    that head's (strided) operands."""
    b, h, r, d = 4096, 4, 1024, 512
    xq, xs, yq, ys = O.make_fp8_einsum_inputs(b, h, r, d, seed=1)
    want = O.fp8_block_einsum_ref(xq, xs, yq, ys, [128, 128])
    x, x_s, y, y_s = xq.to(DEV), xs.to(DEV), yq.to(DEV), ys.to(DEV)
    got = flag_gems.fp8_einsum("bhr,hdr->bhd", x, x_s, y, y_s)
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2 * max(1.0, want.abs().max().item() / 8))
    for head in range(h):
        plain = flag_gems.w8a8_block_fp8_matmul(x[:, head].contiguous(), y[head], x_s[:, head].contiguous(), y_s[head], [128, 128])
        assert torch.equal(got[:, head], plain)


@pytest.mark.parametrize("M", [1, 5, 17, 32, 33, 48, 64, 100, 128])
@pytest.mark.parametrize("B,N,K", [(3, 384, 640), (12, 1024, 2048), (40, 128, 512), (2, 7168, 2304), (10, 1024, 7168), (20, 1024, 1024)])
def test_batches_of_few_rows_go_out_in_one_launch(M, B, N, K):
    """Up to 128 rows per matrix the weight-streaming kernels and the four-stage tile kernel take the whole batch in one
    launch (the entry in the grid, every entry with its own partial sums and counters); strided operands and outputs,
    and a second call on the same workspace.  The last shape has more than 64 MB of weights, which moves 33..64 rows to
    the tile kernel as well; the one after it has enough 16-row groups in all for a wavefront per group (up to 32 rows)."""
    xq, xs, yq, ys = O.make_fp8_einsum_inputs(M, B, K, N, seed=M + B)
    want = O.fp8_block_einsum_ref(xq, xs, yq, ys, [128, 128]).permute(1, 0, 2)       # [B, M, N]
    x, x_s = xq.permute(1, 0, 2).to(DEV), xs.permute(1, 0, 2).to(DEV)                # strided views, as fp8_einsum passes them
    z = torch.full((B, M, N + 3), 3.0, dtype=torch.bfloat16, device=DEV)
    for _ in range(2):
        flag_gems.w8a8_block_fp8_bmm(x, yq.to(DEV), x_s, ys.to(DEV), [128, 128], z=z[:, :, :N])
        top = want.abs().max().item()
        torch.testing.assert_close(z[:, :, :N].cpu().float(), want, rtol=1e-2, atol=1e-2 * max(1.0, top / 8))
        assert torch.all(z[:, :, N:] == 3.0)


@pytest.mark.parametrize("B,M,N,K", [(8, 256, 1024, 4096), (4, 384, 512, 2048), (5, 200, 640, 1024), (16, 130, 1024, 7168)])
def test_batches_above_128_rows_with_few_tiles_in_all(B, M, N, K):
    """While the whole batch has no more 128 x 128 tiles than the GPU has compute units it goes out as one launch of the
    four-stage tile kernel with K split over blocks (64 ... 208 tiles here): against the oracle, rows that end inside a
    tile, and the same bits on a second call."""
    xq, xs, yq, ys = O.make_fp8_einsum_inputs(M, B, K, N, seed=B + M)
    want = O.fp8_block_einsum_ref(xq, xs, yq, ys, [128, 128]).permute(1, 0, 2)       # [B, M, N]
    x, x_s = xq.permute(1, 0, 2).to(DEV), xs.permute(1, 0, 2).to(DEV)
    got = flag_gems.w8a8_block_fp8_bmm(x, yq.to(DEV), x_s, ys.to(DEV), [128, 128])
    top = want.abs().max().item()
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2 * max(1.0, top / 8))
    got32 = flag_gems.w8a8_block_fp8_bmm(x, yq.to(DEV), x_s, ys.to(DEV), [128, 128], output_dtype=torch.float32)
    torch.testing.assert_close(got32.cpu(), want, rtol=1e-4, atol=1e-4 * max(1.0, top))
    again = flag_gems.w8a8_block_fp8_bmm(x, yq.to(DEV), x_s, ys.to(DEV), [128, 128])
    assert torch.equal(again.view(torch.int16), got.view(torch.int16))


def test_bmm_into_callers_buffer_and_other_dtypes():
    B, M, N, K = 3, 200, 384, 512
    xq, xs, yq, ys = O.make_fp8_einsum_inputs(M, B, K, N, seed=2)
    x, x_s = xq.permute(1, 0, 2).contiguous().to(DEV), xs.permute(1, 0, 2).contiguous().to(DEV)
    want = O.fp8_block_einsum_ref(xq, xs, yq, ys, [128, 128]).permute(1, 0, 2)
    for dt, tol in ((torch.float32, 1e-4), (torch.float16, 2e-3), (torch.bfloat16, 1e-2)):
        z = torch.full((B, M, N + 8), 7.0, dtype=dt, device=DEV)
        out = flag_gems.w8a8_block_fp8_bmm(x, yq.to(DEV), x_s, ys.to(DEV), [128, 128], z=z[:, :, :N], output_dtype=dt)
        assert out.data_ptr() == z.data_ptr()
        torch.testing.assert_close(z[:, :, :N].cpu().float(), want, rtol=tol, atol=tol * want.abs().max().item())
        assert torch.all(z[:, :, N:] == 7.0)
    with pytest.raises(AssertionError):
        flag_gems.fp8_einsum("bhr,hrd->bhd", x, x_s, yq.to(DEV), ys.to(DEV))
    with pytest.raises(AssertionError):
        flag_gems.w8a8_block_fp8_bmm(x, yq.to(DEV), x_s, ys.to(DEV), [64, 128])
    assert flag_gems.w8a8_block_fp8_bmm(x[:0], yq[:0].to(DEV), x_s[:0], ys[:0].to(DEV)).shape == (0, M, N)


@pytest.mark.parametrize("ue8m0", [True, False])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_per_token_cast_matches_oracle(ue8m0, dtype):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(300, 1024, generator=g) * torch.exp(2 * torch.randn(300, 1024, generator=g))).to(dtype)
    x[0, :128] = 0.0
    x[1, 130] = float("inf")
    x[2, 5] = float("nan")
    want_q, want_s = O.per_token_cast_to_fp8_ref(x, use_ue8m0=ue8m0)
    q, s = flag_gems.per_token_cast_to_fp8(x.to(DEV), use_ue8m0=ue8m0)
    assert_scales_equal(s, want_s)
    assert_codes_equal(q, want_q)
