"""GPU parity of the quantizer entry points against the CPU oracle: bit-exact codes and scales.

Shapes and parameters follow the reference's own tests (tests/test_act_quant.py:34-40,
tests/accuracy_utils.py:90-96 of the reference); everything goes through the C ABI via the
flag_gems-compatible Python entry points."""
import os

import numpy as np
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O
from tests._util import assert_codes_equal, assert_scales_equal

pytestmark = pytest.mark.gpu
DEV = "cuda"
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _x(shape, seed, kind="randn", dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    if kind == "randn":
        x = torch.randn(*shape, generator=g)
    elif kind == "rand":
        x = torch.rand(*shape, generator=g)
    else:
        x = torch.randn(*shape, generator=g) * torch.exp(3 * torch.randn(*shape, generator=g))
    return x.to(dtype)


@pytest.mark.parametrize("M", [1, 40, 164, 512, 3454])
@pytest.mark.parametrize("N", [128, 896, 2048, 8192])
@pytest.mark.parametrize("block", [64, 128])
@pytest.mark.parametrize("scale_fmt", [None, "ue8m0"])
def test_act_quant_matches_oracle(M, N, block, scale_fmt):
    x = _x((M, N), 0)
    want_y, want_s = O.act_quant_ref(x, block, scale_fmt)
    y, s = flag_gems.act_quant_triton(x.to(DEV), block, scale_fmt)
    assert y.dtype == torch.float8_e4m3fn and y.shape == x.shape
    assert s.dtype == torch.float32 and s.shape == (M, N // block)
    assert_scales_equal(s, want_s, "act_quant scales")
    assert_codes_equal(y, want_y, "act_quant codes")


@pytest.mark.parametrize("kind", ["wide", "rand"])
def test_act_quant_wide_range_and_leading_dims(kind):
    x = _x((3, 5, 1024), 1, kind)
    want_y, want_s = O.act_quant_ref(x, 128)
    y, s = flag_gems.act_quant_triton(x.to(DEV))
    assert y.shape == (3, 5, 1024) and s.shape == (3, 5, 8)
    assert_scales_equal(s, want_s)
    assert_codes_equal(y, want_y)


@pytest.mark.parametrize("num_tokens", [7, 83, 2048])
@pytest.mark.parametrize("d", [512, 4096, 5120, 13824])
@pytest.mark.parametrize("group_size", [64, 128, 256, 512])
@pytest.mark.parametrize("scale_ue8m0", [True, False])
def test_per_token_group_quant_matches_oracle(num_tokens, d, group_size, scale_ue8m0):
    x = _x((num_tokens, d), 0, "rand")
    want_q, want_s = O.per_token_group_quant_fp8_ref(x, group_size, scale_ue8m0=scale_ue8m0)
    q, s = flag_gems.per_token_group_quant_fp8(x.to(DEV), group_size, scale_ue8m0=scale_ue8m0)
    assert_scales_equal(s, want_s, "group quant scales")
    assert_codes_equal(q, want_q, "group quant codes")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("kind", ["randn", "wide"])
@pytest.mark.parametrize("ue8m0", [False, True])
def test_per_token_group_quant_dtypes(dtype, kind, ue8m0):
    x = _x((33, 1024), 2, kind, dtype)
    want_q, want_s = O.per_token_group_quant_fp8_ref(x, 128, scale_ue8m0=ue8m0)
    q, s = flag_gems.per_token_group_quant_fp8(x.to(DEV), 128, scale_ue8m0=ue8m0)
    assert_scales_equal(s, want_s)
    assert_codes_equal(q, want_q)


def test_div_scale_rule_matches_moe_reference():
    x = _x((64, 2048), 3, "wide")
    want_q, want_s = O.per_token_group_quant_fp8_div_ref(x, 128)
    q, s = flag_gems.per_token_group_quant_fp8(x.to(DEV), 128, scale_rule="div")
    assert_scales_equal(s, want_s)
    assert_codes_equal(q, want_q)


def test_column_major_scales_same_values():
    x = _x((83, 1024), 4).to(DEV)
    q0, s0 = flag_gems.per_token_group_quant_fp8(x, 128)
    q1, s1 = flag_gems.per_token_group_quant_fp8(x, 128, column_major_scales=True)
    assert s1.shape == (83, 8) and s1.stride() == (1, 83)
    assert torch.equal(q0.view(torch.uint8), q1.view(torch.uint8))
    assert torch.equal(s0, s1.contiguous())


def test_strided_rows_and_odd_group_sizes():
    base = _x((17, 2048), 5)
    x = base[:, 256 : 256 + 1024]  # row stride 2048, rows still 16-byte aligned
    want_q, want_s = O.per_token_group_quant_fp8_ref(x.contiguous(), 128)
    q, s = flag_gems.per_token_group_quant_fp8(base.to(DEV)[:, 256 : 256 + 1024], 128)
    assert_scales_equal(s, want_s)
    assert_codes_equal(q, want_q)
    # misaligned view (offset by one element) and group sizes the vector kernel does not take
    x = base[:, 1 : 1 + 960]
    for g in (96, 24, 960):
        want_q, want_s = O.per_token_group_quant_fp8_ref(x.contiguous(), g)
        q, s = flag_gems.per_token_group_quant_fp8(base.to(DEV)[:, 1 : 1 + 960], g)
        assert_scales_equal(s, want_s, f"group {g}")
        assert_codes_equal(q, want_q, f"group {g}")


def test_special_values():
    x = _x((8, 512), 6)
    x[0, :128] = 0.0                      # all-zero group: scale comes from the floor
    x[1, 5] = float("nan")                # NaN poisons its group
    x[2, 130] = float("inf")              # Inf: scale inf, finite elements -> 0, Inf -> NaN
    x[3, 300] = -3e38                     # lone huge element
    x[4, :] = 2.0 ** -130                 # denormal-range inputs (below bf16 normal range)
    x[5, 7] = float("-inf")
    for fmt in (None, "ue8m0"):
        want_y, want_s = O.act_quant_ref(x, 128, fmt)
        y, s = flag_gems.act_quant_triton(x.to(DEV), 128, fmt)
        assert_scales_equal(s, want_s, f"act special {fmt}")
        assert_codes_equal(y, want_y, f"act special {fmt}")
    for ue in (False, True):
        want_q, want_s = O.per_token_group_quant_fp8_ref(x, 128, scale_ue8m0=ue)
        q, s = flag_gems.per_token_group_quant_fp8(x.to(DEV), 128, scale_ue8m0=ue)
        assert_scales_equal(s, want_s, f"group special {ue}")
        assert_codes_equal(q, want_q, f"group special {ue}")


def test_every_bf16_value_through_the_converter():
    # a group whose amax is 448 has scale exactly 1.0, so codes are the plain e4m3 cast of x:
    # run all finite bf16 patterns with |x| <= 448 through the kernel
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    v = bits.view(torch.bfloat16)
    keep = v.float().abs() <= 448
    v = v[keep]
    pad = (-v.numel()) % 127
    v = torch.cat([v, torch.zeros(pad, dtype=torch.bfloat16)]).view(-1, 127)
    x = torch.cat([torch.full((v.shape[0], 1), 448.0, dtype=torch.bfloat16), v], dim=1).contiguous()
    want_y, want_s = O.act_quant_ref(x, 128)
    assert torch.all(want_s == 1.0)
    y, s = flag_gems.act_quant_triton(x.to(DEV), 128)
    assert_scales_equal(s, want_s)
    assert_codes_equal(y, want_y)
    assert_codes_equal(y, x.float().to(torch.float8_e4m3fn))


def test_golden_vectors():
    z = np.load(os.path.join(GOLD, "config1.npz"))
    x, _ = O.make_config1(0)
    y, s = flag_gems.act_quant_triton(x.to(DEV), 128)
    assert np.array_equal(y.cpu().view(torch.uint8).numpy(), z["xq"])
    assert np.array_equal(s.cpu().numpy().view(np.uint32), z["xs"].view(np.uint32))
    v = np.load(os.path.join(GOLD, "quant_variants.npz"))
    for name, fn in [
        ("group", lambda t: flag_gems.per_token_group_quant_fp8(t, 128)),
        ("group_ue8m0", lambda t: flag_gems.per_token_group_quant_fp8(t, 128, scale_ue8m0=True)),
        ("act_ue8m0", lambda t: flag_gems.act_quant_triton(t, 128, "ue8m0")),
        ("div", lambda t: flag_gems.per_token_group_quant_fp8(t, 128, scale_rule="div")),
    ]:
        q, sc = fn(x.to(DEV))
        assert np.array_equal(q.cpu().view(torch.uint8).numpy(), v[name + "_q"]), name
        assert np.array_equal(sc.cpu().numpy().view(np.uint32), v[name + "_s"].view(np.uint32)), name


def test_full_size_properties():
    # largest shape of the reference's grid: 38594 x 8192 bf16 (632 MB); properties only
    torch.manual_seed(0)
    x = torch.randn(38594, 8192, device=DEV, dtype=torch.bfloat16)
    y, s = flag_gems.act_quant_triton(x, 128)
    xg = x.view(38594, 64, 128)
    amax = xg.abs().amax(-1).float().clamp(min=1e-4)
    assert torch.equal(s, amax * torch.tensor(1.0 / 448.0, device=DEV))
    idx = xg.abs().argmax(-1, keepdim=True)
    top = y.view(torch.uint8).view(38594, 64, 128).gather(-1, idx)
    assert torch.all((top & 0x7F) == 0x7E)
    yn, sn = flag_gems.act_quant_triton(-x, 128)
    assert torch.equal(sn, s)
    assert torch.equal(yn.view(torch.uint8), y.view(torch.uint8) ^ 0x80)


def test_vllm_op_writes_callers_buffers():
    flag_gems.patch_empty_vllm()
    x = _x((83, 1024), 7).to(DEV)
    q = torch.empty(83, 1024, dtype=torch.float8_e4m3fn, device=DEV)
    for col_major in (False, True):
        s = torch.empty(8, 83, dtype=torch.float32, device=DEV).t() if col_major else torch.empty(83, 8, dtype=torch.float32, device=DEV)
        torch.ops._C.per_token_group_fp8_quant(x, q, s, 128, 1e-10, -448.0, 448.0, False)
        want_q, want_s = O.per_token_group_quant_fp8_ref(x.cpu(), 128)
        assert_scales_equal(s, want_s)
        assert_codes_equal(q, want_q)


def test_process_wide_rule_selects_the_kernels_formula():
    """set_group_quant_rule("kernel"): the default of per_token_group_quant_fp8, of the fused producers and of the
    vLLM operator becomes the reference's device-kernel arithmetic (fp32 floor, amax / 448, true division:
    src/flag_gems/ops/per_token_group_quant_fp8.py:55-70); "test_reference" is the torch helper's.  Both against
    their formulas, bit for bit; a group of zeros shows the floor, which is where the fp32 and the bf16 eps differ."""
    flag_gems.patch_empty_vllm()
    x = _x((61, 1024), 11)
    x[3, 128:256] = 0
    x[:, 512:640] *= 1e-9
    xd = x.to(DEV)
    assert flag_gems.get_group_quant_rule() == "test_reference"
    try:
        for rule, ref in (("kernel", O.per_token_group_quant_fp8_kernel_ref), ("test_reference", O.per_token_group_quant_fp8_ref)):
            flag_gems.set_group_quant_rule(rule)
            for ue8m0 in (False, True):
                want_q, want_s = ref(x, 128, scale_ue8m0=ue8m0)
                q, s = flag_gems.per_token_group_quant_fp8(xd, 128, scale_ue8m0=ue8m0)
                assert_scales_equal(s, want_s, f"{rule} ue8m0={ue8m0}")
                assert_codes_equal(q, want_q, f"{rule} ue8m0={ue8m0}")
                q2 = torch.empty_like(q)
                s2 = torch.empty_like(s)
                torch.ops._C.per_token_group_fp8_quant(xd, q2, s2, 128, 1e-10, -448.0, 448.0, ue8m0)
                assert_scales_equal(s2, want_s, f"vLLM op, {rule}")
                assert_codes_equal(q2, want_q, f"vLLM op, {rule}")
        flag_gems.set_group_quant_rule("kernel")
        # an explicit scale_rule keeps its own meaning whatever the default is
        want_q, want_s = O.per_token_group_quant_fp8_div_ref(x, 128)
        q, s = flag_gems.per_token_group_quant_fp8(xd, 128, scale_rule="div")
        assert_scales_equal(s, want_s)
        assert_codes_equal(q, want_q)
    finally:
        flag_gems.set_group_quant_rule("test_reference")
    with pytest.raises(ValueError):
        flag_gems.set_group_quant_rule("fast")


def test_empty_inputs():
    y, s = flag_gems.act_quant_triton(torch.empty(0, 256, dtype=torch.bfloat16, device=DEV))
    assert y.shape == (0, 256) and s.shape == (0, 2)
    q, s = flag_gems.per_token_group_quant_fp8(torch.empty(0, 256, dtype=torch.bfloat16, device=DEV), 128)
    assert q.shape == (0, 256) and s.shape == (0, 2)


def test_power_of_two_scales_next_to_the_powers_of_two():
    """scale_ue8m0 rounds the scale up to a power of two through ceil(log2(s)) with an fp32 logarithm, which rounds
    the logarithm of a scale a few steps above 2^n down to n: the kernel decides that case from the bits of the scale.
    Rows whose maximum walks step by step across 448 * 2^n, for every n the rule distinguishes, against the oracle."""
    import numpy as np
    rows = []
    for n in list(range(-33, 40)) + [60, 64, 65, 100, 119]:
        base = np.array([448.0 * 2.0 ** n], dtype=np.float32).view(np.uint32)[0]
        for step in range(-6, 60):
            rows.append(np.uint32(int(base) + step))
    amax = torch.from_numpy(np.array(rows, dtype=np.uint32).view(np.float32).copy())
    assert torch.isfinite(amax).all()
    g = torch.Generator().manual_seed(0)
    x = (torch.rand(amax.numel(), 128, generator=g) * 2 - 1) * amax[:, None] * 0.5
    x[:, 17] = -amax
    for gs, xx in ((128, x), (64, x[:, 8:72].contiguous())):
        want_q, want_s = O.per_token_group_quant_fp8_ref(xx, gs, scale_ue8m0=True)
        q, s = flag_gems.per_token_group_quant_fp8(xx.to(DEV), gs, scale_ue8m0=True)
        assert torch.equal(s.cpu().view(torch.int32), want_s.view(torch.int32))
        assert torch.equal(q.cpu().view(torch.uint8), want_q.view(torch.uint8))
    # the scales are powers of two, and both sides of every boundary were visited
    assert (want_s.view(torch.int32) & 0x7FFFFF).eq(0).all()
