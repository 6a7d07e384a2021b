"""GPU parity of RMSNorm (with and without the residual add) alone and fused into the per-token-group FP8 quantizer.

Bars.  (1) The norm operators against the CPU oracle, which restates the reference's kernels
(src/flag_gems/ops/rms_norm.py:54-66, src/flag_gems/fused/fused_add_rms_norm.py:92-118) with the library's documented
order of the sum of squares: bit-exact (normalised rows and the updated residual).  (2) The fused call against the
oracle chain norm -> per_token_group_quant_fp8: codes and scales bit-exact.  (3) The fused call against the
library's own two separate calls: bit-exact, for every dtype, group size, rule and layout."""
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O
from tests._util import assert_codes_equal, assert_scales_equal

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _data(rows, cols, seed, dtype, scale=1.5):
    g = torch.Generator().manual_seed(seed)
    x = (scale * torch.randn(rows, cols, generator=g)).to(dtype)
    r = (2.0 * torch.randn(rows, cols, generator=g)).to(dtype)
    w = (1 + 0.25 * torch.randn(cols, generator=g)).to(dtype)
    return x, r, w


def _same_bits(got, want, what):
    g, w = got.cpu(), want.cpu()
    same = (g == w) | (g.isnan() & w.isnan())
    assert bool(same.all()), f"{what}: {(~same).sum().item()} of {g.numel()} differ, first at {(~same).nonzero()[0].tolist()}"
    # signed zeros too
    assert torch.equal(torch.signbit(g) & ~g.isnan(), torch.signbit(w) & ~w.isnan()), f"{what}: sign of a zero"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,cols", [(1, 128), (3, 8), (17, 2048), (5, 2056), (64, 4096), (33, 7168), (4500, 1024),
                                       (9, 16384)])
def test_rms_norm_is_the_oracles_bit_for_bit(dtype, rows, cols):
    x, r, w = _data(rows, cols, rows + cols, dtype)
    for eps in (1e-5, 1e-6):
        got = flag_gems.rms_norm(x.to(DEV), (cols,), w.to(DEV), eps)
        _same_bits(got, O.rms_norm_ref(x, w, eps), f"rms_norm {dtype} {rows}x{cols} eps {eps}")
    xd, rd = x.to(DEV), r.to(DEV)
    out, res = flag_gems.fused_add_rms_norm(xd, rd, (cols,), w.to(DEV), 1e-6)
    assert out.data_ptr() == xd.data_ptr() and res.data_ptr() == rd.data_ptr()   # in place, as the reference
    want_y, want_r = O.fused_add_rms_norm_ref(x, r, w, 1e-6)
    _same_bits(res, want_r, f"residual {dtype} {rows}x{cols}")
    _same_bits(out, want_y, f"fused_add_rms_norm {dtype} {rows}x{cols}")


def test_leading_dimensions_and_empty_inputs():
    x, r, w = _data(6 * 5, 512, 7, torch.bfloat16)
    got = flag_gems.rms_norm(x.view(6, 5, 512).to(DEV), (512,), w.to(DEV))
    _same_bits(got.view(30, 512), O.rms_norm_ref(x, w), "3-D input")
    assert got.shape == (6, 5, 512)
    empty = torch.empty((0, 512), dtype=torch.bfloat16, device=DEV)
    assert flag_gems.rms_norm(empty, (512,), w.to(DEV)).shape == (0, 512)
    q, s = flag_gems.rms_norm_per_token_group_quant_fp8(empty, w.to(DEV), 128)
    assert q.shape == (0, 512) and s.shape == (0, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("group", [64, 128])
@pytest.mark.parametrize("with_residual", [False, True])
def test_fused_is_the_oracle_chain_bit_for_bit(dtype, group, with_residual):
    for (rows, cols), seed in (((40, 2048), 1), ((7, 7168), 2), ((300, 1152), 3)):
        x, r, w = _data(rows, cols, seed, dtype, scale=3.0)
        if with_residual:
            y, want_r = O.fused_add_rms_norm_ref(x, r, w, 1e-6)
        else:
            y, want_r = O.rms_norm_ref(x, w, 1e-6), None
        want_q, want_s = O.per_token_group_quant_fp8_ref(y, group)
        rd = r.to(DEV) if with_residual else None
        xd = x.to(DEV)
        q, s = flag_gems.rms_norm_per_token_group_quant_fp8(xd, w.to(DEV), group, eps=1e-6, residual=rd)
        what = f"{dtype} group {group} residual {with_residual} {rows}x{cols}"
        assert_scales_equal(s, want_s, what)
        assert_codes_equal(q, want_q, what)
        assert torch.equal(xd.cpu(), x), "the fused call must not write its input"
        if with_residual:
            _same_bits(rd, want_r, what + " residual")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fused_equals_the_two_separate_calls_rules_and_layouts(dtype):
    x, r, w = _data(600, 4096, 11, dtype, scale=4.0)
    x[0] = 0.0                              # a zero row: y = 0, every scale from the floor
    x[1, 5] = float("nan")                  # NaN spreads over its row through the variance
    x[2, 700] = float("inf")                # infinite variance: rrms = 0, the row becomes 0 and NaN
    x[3] = x[3] * 1e-3
    xd, wd = x.to(DEV), w.to(DEV)
    y = flag_gems.rms_norm(xd, (4096,), wd, 1e-5)
    for kwargs in ({}, {"column_major_scales": True}, {"scale_rule": "div"}, {"scale_ue8m0": True},
                   {"dtype": torch.float8_e5m2}):
        for group in (32, 128, 512):
            qk = dict(kwargs)
            want_q, want_s = flag_gems.per_token_group_quant_fp8(y, group, **qk)
            q, s = flag_gems.rms_norm_per_token_group_quant_fp8(xd, wd, group, eps=1e-5, **qk)
            assert s.stride() == want_s.stride() and q.shape == want_q.shape
            assert_scales_equal(s, want_s, f"{kwargs} group {group}")
            assert_codes_equal(q, want_q, f"{kwargs} group {group}")
    # with the residual: the separate call works in place on copies
    x2, r2 = xd.clone(), r.to(DEV)
    r_fused = r2.clone()
    flag_gems.fused_add_rms_norm(x2, r2, (4096,), wd, 1e-5)
    want_q, want_s = flag_gems.per_token_group_quant_fp8(x2, 128)
    q, s = flag_gems.rms_norm_per_token_group_quant_fp8(xd, wd, 128, eps=1e-5, residual=r_fused)
    assert_scales_equal(s, want_s, "residual")
    assert_codes_equal(q, want_q, "residual")
    _same_bits(r_fused, r2, "residual update")


def test_full_size_properties():
    """[4096, 7168] bf16, the bench's shape: too big for the oracle's loop in seconds, so size-independent properties.
    Unit weight, eps = 0: dequantised rows have unit mean square (to fp8 accuracy), every scale is amax / 448 of a
    value whose largest element is below sqrt(cols), and scaling x by a power of two changes nothing at all."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(4096, 7168, generator=g).bfloat16().to(DEV)
    w = torch.ones(7168, dtype=torch.bfloat16, device=DEV)
    q, s = flag_gems.rms_norm_per_token_group_quant_fp8(x, w, 128, eps=0.0)
    deq = q.float().view(4096, 56, 128) * s[:, :, None]
    ms = (deq.double() ** 2).mean((1, 2))
    assert float((ms - 1).abs().max()) < 2e-2       # e4m3 keeps 3 mantissa bits: a few per cent per element, averaged
    assert float(s.max()) * 448 < 7168 ** 0.5 and float(s.min()) > 0
    q2, s2 = flag_gems.rms_norm_per_token_group_quant_fp8(x * 4, w, 128, eps=0.0)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2, s)


def test_unsupported_requests_fail_loudly():
    x = torch.zeros((4, 16392), dtype=torch.bfloat16, device=DEV)
    w = torch.ones(16392, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="at most 16384"):
        flag_gems.rms_norm(x, (16392,), w)
    x = torch.zeros((4, 132), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        flag_gems.rms_norm(x, (132,), torch.ones(132, dtype=torch.bfloat16, device=DEV))
    x = torch.zeros((4, 256), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(NotImplementedError):
        flag_gems.rms_norm(x, (256,), torch.ones(256, dtype=torch.float32, device=DEV))
    with pytest.raises(RuntimeError, match="group size"):
        flag_gems.rms_norm_per_token_group_quant_fp8(x, torch.ones(256, dtype=torch.bfloat16, device=DEV), 4)


def test_vllm_rms_norm_and_silu_and_mul_write_the_callers_tensors():
    """_C::rms_norm(result, input, weight, epsilon) and _C::silu_and_mul(out, input): the same bits as the operators
    that allocate, in the tensor the caller passed."""
    flag_gems.patch_empty_vllm()
    g = torch.Generator().manual_seed(17)
    for dtype in (torch.bfloat16, torch.float16):
        x = torch.randn(3, 37, 1024, generator=g).to(dtype).to(DEV)
        w = (1 + 0.1 * torch.randn(1024, generator=g)).to(dtype).to(DEV)
        result = torch.full_like(x, 7.0)
        assert torch.ops._C.rms_norm(result, x, w, 1e-6) is None
        assert torch.equal(result, flag_gems.rms_norm(x, (1024,), w, 1e-6))
        want = O.rms_norm_ref(x.cpu().reshape(-1, 1024), w.cpu(), 1e-6)
        assert torch.equal(result.cpu().reshape(-1, 1024).view(torch.int16), want.view(torch.int16))
        out = torch.full((3, 37, 512), 7.0, dtype=dtype, device=DEV)
        assert torch.ops._C.silu_and_mul(out, x) is None
        assert torch.equal(out, flag_gems.silu_and_mul_packed(x))
    with pytest.raises(AssertionError):
        flag_gems.silu_and_mul_packed_out(torch.empty(3, 37, 500, dtype=torch.float16, device=DEV), x)
    with pytest.raises(AssertionError):
        flag_gems.rms_norm_out(torch.empty(3, 37, 512, dtype=torch.float16, device=DEV), x, (1024,), w)
