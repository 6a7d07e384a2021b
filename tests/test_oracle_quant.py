"""Pins the quantizer functions of oracle/fp8_linear_oracle.py.

Checks: a numpy brute-force quantizer built on the bit-level encoder of
oracle/e4m3.py, hand-worked known answers, and invariants that hold for any
seed.  Reference functions restated by the oracle are cited there."""
import numpy as np
import pytest
import torch

from oracle import e4m3
from oracle import fp8_linear_oracle as O

F32 = np.float32


def _brute_quant(x_f32: np.ndarray, group: int, floor: float, scale_rule: str, quot_rule: str, ue8m0: str = "none"):
    """Scalar loops over groups; IEEE float32 arithmetic through numpy scalars."""
    rows, cols = x_f32.shape
    codes = np.zeros((rows, cols), dtype=np.uint8)
    scales = np.zeros((rows, cols // group), dtype=np.float32)
    inv448 = F32(1.0) / F32(448.0)
    for r in range(rows):
        for g in range(cols // group):
            seg = x_f32[r, g * group : (g + 1) * group]
            amax = F32(0.0)
            for v in seg:
                av = F32(abs(v))
                if np.isnan(av) or av > amax:
                    amax = av
                    if np.isnan(av):
                        break
            if not np.isnan(amax) and amax < F32(floor):
                amax = F32(floor)
            s = amax * inv448 if scale_rule == "mul" else amax / F32(448.0)
            if ue8m0 == "bits":
                b = np.array([s], dtype=np.float32).view(np.uint32)[0]
                e = ((b >> 23) & 0xFF) + (1 if b & 0x7FFFFF else 0)
                s = np.array([e << 23], dtype=np.uint32).view(np.float32)[0]
            elif ue8m0 == "log2":
                s = F32(2.0) ** F32(np.ceil(np.log2(max(abs(s), F32(1e-10)))))
            if quot_rule == "recip":
                q = seg * (F32(1.0) / s)
            else:
                q = seg / s
            q = np.minimum(np.maximum(q, F32(-448.0)), F32(448.0))  # propagates NaN
            codes[r, g * group : (g + 1) * group] = e4m3.encode(q.astype(np.float32))
            scales[r, g] = s
    return codes, scales


def _rand_bf16(rows, cols, seed, kind="randn"):
    g = torch.Generator().manual_seed(seed)
    if kind == "randn":
        x = torch.randn(rows, cols, generator=g)
    elif kind == "rand":
        x = torch.rand(rows, cols, generator=g)
    else:  # heavy tailed, spans many binades
        x = torch.randn(rows, cols, generator=g) * torch.exp(3 * torch.randn(rows, cols, generator=g))
    return x.bfloat16()


@pytest.mark.parametrize("kind", ["randn", "rand", "wide"])
@pytest.mark.parametrize("group", [64, 128])
def test_act_quant_ref_vs_brute_force(kind, group):
    x = _rand_bf16(6, 512, 3, kind)
    y, s = O.act_quant_ref(x, group)
    codes, scales = _brute_quant(x.float().numpy(), group, 1e-4, "mul", "recip")
    assert np.array_equal(y.view(torch.uint8).numpy(), codes)
    assert np.array_equal(s.numpy().view(np.uint32), scales.view(np.uint32))


@pytest.mark.parametrize("kind", ["randn", "wide"])
def test_act_quant_ref_ue8m0_vs_brute_force(kind):
    x = _rand_bf16(5, 384, 4, kind)
    y, s = O.act_quant_ref(x, 128, "ue8m0")
    codes, scales = _brute_quant(x.float().numpy(), 128, 1e-4, "mul", "recip", "bits")
    assert np.array_equal(y.view(torch.uint8).numpy(), codes)
    assert np.array_equal(s.numpy().view(np.uint32), scales.view(np.uint32))
    # a power of two in [raw, 2*raw)
    raw = x.float().view(5, 3, 128).abs().amax(-1).clamp(min=1e-4) * (1.0 / 448.0)
    assert torch.all(s >= raw) and torch.all(s < 2 * raw)
    assert torch.all((s.view(torch.int32) & 0x7FFFFF) == 0)


@pytest.mark.parametrize("kind", ["randn", "rand", "wide"])
@pytest.mark.parametrize("group", [64, 128, 256])
@pytest.mark.parametrize("ue8m0", [False, True])
def test_group_quant_ref_vs_brute_force(kind, group, ue8m0):
    x = _rand_bf16(4, 512, 5, kind)
    y, s = O.per_token_group_quant_fp8_ref(x, group, scale_ue8m0=ue8m0)
    # bf16 amax then widening equals fp32 amax of the widened values (max is exact);
    # the eps floor is applied in bf16: bf16(1e-10)
    floor = float(torch.tensor(1e-10, dtype=torch.bfloat16).float())
    codes, scales = _brute_quant(x.float().numpy(), group, floor, "mul", "div", "log2" if ue8m0 else "none")
    assert np.array_equal(y.view(torch.uint8).numpy(), codes)
    assert np.array_equal(s.numpy().view(np.uint32), scales.view(np.uint32))


def test_group_quant_div_ref_vs_brute_force():
    x = _rand_bf16(4, 512, 6, "wide")
    y, s = O.per_token_group_quant_fp8_div_ref(x, 128)
    floor = float(torch.tensor(1e-10, dtype=torch.bfloat16).float())
    codes, scales = _brute_quant(x.float().numpy(), 128, floor, "div", "div")
    assert np.array_equal(y.view(torch.uint8).numpy(), codes)
    assert np.array_equal(s.numpy().view(np.uint32), scales.view(np.uint32))


@pytest.mark.parametrize("kind", ["randn", "wide"])
def test_group_quant_kernel_ref_vs_brute_force(kind):
    """The device kernel's formula: fp32 floor, amax / 448, true division.  A row of zeros shows the floor: with
    bf16 inputs the torch helper floors at bf16(1e-10), the kernel at fp32(1e-10)."""
    x = _rand_bf16(4, 512, 8, kind)
    x[1, :128] = 0
    y, s = O.per_token_group_quant_fp8_kernel_ref(x, 128)
    codes, scales = _brute_quant(x.float().numpy(), 128, 1e-10, "div", "div")
    assert np.array_equal(y.view(torch.uint8).numpy(), codes)
    assert np.array_equal(s.numpy().view(np.uint32), scales.view(np.uint32))
    assert s[1, 0].item() == np.float32(1e-10) / np.float32(448.0)
    _, s_helper = O.per_token_group_quant_fp8_div_ref(x, 128)
    assert s_helper[1, 0].item() != s[1, 0].item()


def test_mul_and_div_scale_rules_really_differ():
    # the two scale formulas disagree in the last bit for about half of all amax
    # values, so a test that passes with the wrong rule would show here
    amax = torch.arange(0x3C00, 0x4400, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    a = amax * torch.tensor(1.0 / 448.0)
    b = amax / 448.0
    frac = (a != b).float().mean().item()
    assert 0.3 < frac < 0.8


def test_known_answers_unit_scale_group():
    # amax 448 -> scale = 448 * fp32(1/448) = 1.0 exactly, so codes are the plain cast
    vals = [448.0, 224.0, 1.0, 0.30078125, -17.25, 0.0, -0.0, 2.0 ** -9]
    x = torch.zeros(1, 128)
    x[0, : len(vals)] = torch.tensor(vals)
    x = x.bfloat16()
    want = [0x7E, 0x76, 0x38, 0x2A, 0xD9, 0x00, 0x80, 0x01]
    for fn in (lambda t: O.act_quant_ref(t, 128), lambda t: O.per_token_group_quant_fp8_ref(t, 128)):
        y, s = fn(x)
        assert s.item() == 1.0
        assert list(y.view(torch.uint8)[0, : len(vals)].numpy()) == want


def test_special_cases():
    x = torch.zeros(2, 256).bfloat16()
    y, s = O.act_quant_ref(x, 128)
    assert torch.all(y.view(torch.uint8) == 0)
    assert torch.all(s == torch.tensor(1e-4) * torch.tensor(1.0 / 448.0))
    y, s = O.per_token_group_quant_fp8_ref(x, 128)
    assert torch.all(y.view(torch.uint8) == 0)
    assert torch.all(s == torch.tensor(1e-10, dtype=torch.bfloat16).float() * torch.tensor(1.0 / 448.0))
    # NaN poisons its own group only
    x = torch.ones(1, 256).bfloat16()
    x[0, 5] = float("nan")
    y, s = O.act_quant_ref(x, 128)
    assert torch.isnan(s[0, 0]) and not torch.isnan(s[0, 1])
    assert torch.all((y.view(torch.uint8)[0, :128] & 0x7F) == 0x7F)
    assert torch.all(y.view(torch.uint8)[0, 128:] == 0x7E)
    # Inf: scale inf, finite elements -> 0, the Inf itself -> NaN (inf * 0)
    x = torch.ones(1, 128).bfloat16()
    x[0, 7] = float("inf")
    y, s = O.act_quant_ref(x, 128)
    assert torch.isinf(s[0, 0])
    c = y.view(torch.uint8)[0]
    assert c[7] & 0x7F == 0x7F and c[0] == 0
    # lone huge element: everything else flushes to zero, the element itself is 448
    x = torch.full((1, 128), 1e-3).bfloat16()
    x[0, 100] = -3e38
    y, s = O.act_quant_ref(x, 128)
    c = y.view(torch.uint8)[0]
    assert c[100] == 0xFE and torch.all(c[:100] == 0)


@pytest.mark.parametrize("fn", ["act", "group", "div"])
def test_invariants(fn):
    x = _rand_bf16(64, 1024, 7, "wide")
    f = {
        "act": lambda t: O.act_quant_ref(t, 128),
        "group": lambda t: O.per_token_group_quant_fp8_ref(t, 128),
        "div": lambda t: O.per_token_group_quant_fp8_div_ref(t, 128),
    }[fn]
    y, s = f(x)
    yn, sn = f(-x)
    assert torch.equal(s, sn)
    assert torch.equal(y.view(torch.uint8) ^ 0x80, yn.view(torch.uint8))
    # the max-magnitude element of every group encodes to +-448
    xg = x.float().view(64, 8, 128)
    idx = xg.abs().argmax(-1, keepdim=True)
    top = y.view(torch.uint8).view(64, 8, 128).gather(-1, idx)
    assert torch.all((top & 0x7F) == 0x7E)
    # dequantised value within half an fp8 step of x/s (step <= 2**-4 relative, 2**-10 absolute)
    q = xg / s.unsqueeze(-1)
    d = y.float().view(64, 8, 128)
    err = (d - q).abs()
    assert torch.all(err <= torch.maximum(q.abs() * 2.0 ** -4, torch.tensor(2.0 ** -10)) * 1.0001)
    # row order does not matter
    perm = torch.randperm(64, generator=torch.Generator().manual_seed(0))
    yp, sp = f(x[perm].contiguous())
    assert torch.equal(sp, s[perm]) and torch.equal(yp.view(torch.uint8), y.view(torch.uint8)[perm])


def test_per_block_cast_vs_brute_force():
    g = torch.Generator().manual_seed(8)
    w = (0.02 * torch.randn(200, 300, generator=g)).bfloat16()
    wq, ws = O.per_block_cast_to_fp8_ref(w)
    assert wq.shape == (200, 300) and ws.shape == (2, 3)
    wn = w.float().numpy()
    for bi in range(2):
        for bj in range(3):
            blk = wn[bi * 128 : (bi + 1) * 128, bj * 128 : (bj + 1) * 128]
            amax = max(F32(np.abs(blk).max()), F32(1e-4))
            sf = F32(amax) / F32(448.0)
            assert ws[bi, bj].item() == sf
            codes = e4m3.encode((blk * (F32(1.0) / sf)).astype(np.float32))
            got = wq.view(torch.uint8).numpy()[bi * 128 : (bi + 1) * 128, bj * 128 : (bj + 1) * 128]
            assert np.array_equal(codes, got)


def test_per_token_cast_matches_group_quant_shape_and_scale():
    x = _rand_bf16(5, 300, 9)
    xq, sf = O.per_token_cast_to_fp8_ref(x, use_ue8m0=False)
    assert xq.shape == (5, 300) and sf.shape == (5, 3)
    amax = torch.zeros(5, 384)
    amax[:, :300] = x.float()
    want = amax.view(5, 3, 128).abs().amax(-1).clamp(1e-4) / 448.0
    assert torch.equal(sf, want)


# ---- activation between the two GEMMs of an expert / MLP layer


def test_silu_and_mul_ref_pinned():
    g = torch.Generator().manual_seed(41)
    x = (3 * torch.randn(64, 512, generator=g)).bfloat16()
    got = O.silu_and_mul_ref(x)
    gate, up = x[:, :256].double(), x[:, 256:].double()
    exact = gate / (1 + torch.exp(-gate)) * up
    # one rounding of a bf16 result: at most half a step from the exact value (plus fp32 noise far below that)
    step = torch.maximum(exact.abs(), torch.tensor(2.0 ** -126, dtype=torch.float64)) * 2.0 ** -7  # a bf16 step is at most 2^-7 of the value
    assert torch.all((got.double() - exact).abs() <= 0.5 * step + 1e-30)
    # a different formula for the same function
    other = (x[:, :256].float() * torch.sigmoid(x[:, :256].float()) * x[:, 256:].float())
    torch.testing.assert_close(got.float(), other, rtol=2.0 ** -7, atol=1e-30)
    # special cases
    sp = torch.tensor([[0.0, 100.0, -100.0, 3.0, -3.0, 1.0, 2.0, 1.0, 1.0, 1.0]], dtype=torch.float32)
    out = O.silu_and_mul_ref(sp)
    assert out[0, 0] == 0.0 and out[0, 1] == 200.0 and out[0, 2] == 0.0 and torch.signbit(out[0, 2])
    torch.testing.assert_close(out[0, 3] - out[0, 4], torch.tensor(3.0), rtol=1e-6, atol=0)
    assert O.silu_and_mul_ref(torch.zeros(2, 0)).shape == (2, 0)


def test_three_operation_division_is_the_correctly_rounded_quotient():
    """The quantizer kernels replace x / s by q0 = RN(x r), e = RN(x - q0 s) (one fused multiply-add),
    RN(q0 + e r) with r = RN(1 / s), for scales in [2^-60, 2^100].  Emulated here in numpy (float64 holds the
    products of two fp32 values exactly) against fp32 division, on quotients spread over the fp8 range and on
    quotients within a few fp32 steps of the fp8 rounding boundaries."""
    rng = np.random.default_rng(0)
    n = 1_500_000
    for mode in (0, 1):
        s = (np.exp2(rng.uniform(-60, 60, n)) * rng.uniform(1, 2, n)).astype(np.float32)
        if mode == 0:
            x = (s.astype(np.float64) * rng.uniform(-448, 448, n)).astype(np.float32)
        else:
            mid = (rng.integers(16, 32, n) + 0.5) / 16.0 * np.exp2(rng.integers(-10, 9, n))
            x = (s.astype(np.float64) * mid * (1 + rng.integers(-3, 4, n) * 2.0 ** -24)).astype(np.float32)
        want = (x / s).astype(np.float32)
        r = (np.float32(1.0) / s).astype(np.float32)
        q0 = (x * r).astype(np.float32)
        # the fused multiply-add rounds the exact remainder once (it fits fp32 whenever q0 is within a step)
        e = (x.astype(np.float64) - q0.astype(np.float64) * s.astype(np.float64)).astype(np.float32)
        q1 = (q0.astype(np.float64) + e.astype(np.float64) * r.astype(np.float64)).astype(np.float32)
        assert np.array_equal(q1, want)


def test_fast_index_division_is_exact():
    """The quantizer kernel splits a group index n < 2^24 into (row, column) with q = uint(fp32(n) * fp32(1 / d)) and one
    corrective step from the remainder, instead of a 32-bit division.  Emulated here in numpy against integer
    division: every d up to 4096 at the n next to multiples of d and at the top of the range, and random (n, d)."""
    rng = np.random.default_rng(1)

    def fast(n, d):
        inv = (np.float32(1.0) / d.astype(np.float32)).astype(np.float32)
        q = (n.astype(np.float32) * inv).astype(np.float32).astype(np.int64)
        r = n.astype(np.int64) - q * d.astype(np.int64)
        low, high = r < 0, r >= d
        q = q - low + (high & ~low)
        return q, n.astype(np.int64) - q * d.astype(np.int64)

    top = (1 << 24) - 1
    for d0 in range(1, 4097):
        mult = (rng.integers(0, top // d0 + 1, 64) * d0).astype(np.int64)
        n = np.unique(np.clip(np.concatenate([mult - 1, mult, mult + 1, [top, top - 1, 0, d0 - 1]]), 0, top))
        d = np.full_like(n, d0)
        q, r = fast(n, d)
        assert np.array_equal(q, n // d0) and np.array_equal(r, n % d0), d0
    d = rng.integers(1, 1 << 23, 2_000_000)
    n = rng.integers(0, 1 << 24, 2_000_000)
    q, r = fast(n, d)
    assert np.array_equal(q, n // d) and np.array_equal(r, n % d)
    # multiples of large divisors, where the product lands next to an integer
    k = rng.integers(1, 64, 500_000)
    d = rng.integers(1 << 10, 1 << 18, 500_000)
    n = np.minimum(k * d + rng.integers(-1, 2, 500_000), top)
    q, r = fast(n, d)
    assert np.array_equal(q, n // d) and np.array_equal(r, n % d)


# ---- DeepGEMM-style helpers (inputs of the batched GEMM and of the weight quantizer)


def test_ceil_to_ue8m0_is_the_least_power_of_two_not_below():
    """The smallest power of two >= |s|, held in [2^-126, 2^127]: checked with math.frexp (no bit tricks) on
    random scales over the whole exponent range, on exact powers of two (which must map to themselves: a floor
    would pass "is a power of two" but not this), on their neighbours, and at the clamp edges."""
    import math

    rng = np.random.default_rng(3)
    s = (np.exp2(rng.uniform(-126, 127, 20000)) * rng.choice([-1.0, 1.0], 20000)).astype(np.float32)
    pw = np.exp2(np.arange(-126, 128)).astype(np.float32)
    up = np.nextafter(pw, np.float32(np.inf)).astype(np.float32)
    down = np.nextafter(pw, np.float32(0)).astype(np.float32)
    vals = np.concatenate([s, pw, -pw, up, down[1:]])
    got = O._ceil_to_ue8m0(torch.from_numpy(vals)).numpy()
    for v, g in zip(vals.tolist(), got.tolist()):
        m, e = math.frexp(abs(v))                 # |v| = m * 2^e, 0.5 <= m < 1
        want = 2.0 ** (e - 1) if m == 0.5 else 2.0 ** e
        want = min(max(want, 2.0 ** -126), 2.0 ** 127)
        assert g == want, (v, g, want)
        assert g >= min(abs(v), 2.0 ** 127) and (g < 2 * abs(v) or g == 2.0 ** -126)
    # clamp edges: zero and subnormals go to the smallest normal, Inf and NaN (exponent field 255) to 2^127
    edge = torch.tensor([0.0, -0.0, 1e-45, 1.1e-38, float("inf"), float("-inf"), float("nan"), 3.4e38])
    out = O._ceil_to_ue8m0(edge).tolist()
    assert out[:4] == [2.0 ** -126] * 4 and out[4:] == [2.0 ** 127] * 4


@pytest.mark.parametrize("use_ue8m0", [False, True])
def test_per_token_cast_codes_vs_brute_force(use_ue8m0):
    """Codes and scales of per_token_cast_to_fp8_ref against numpy scalar arithmetic and the bit-level encoder:
    ragged last group (zero padding takes part in no maximum that matters and yields no code), both scale kinds."""
    x = _rand_bf16(6, 300, 21, "wide")
    xq, sf = O.per_token_cast_to_fp8_ref(x, use_ue8m0=use_ue8m0)
    assert xq.shape == (6, 300) and sf.shape == (6, 3)
    xn = x.float().numpy()
    for r in range(6):
        for g in range(3):
            seg = xn[r, g * 128 : min((g + 1) * 128, 300)]
            amax = max(F32(np.abs(seg).max()), F32(1e-4))
            s = F32(amax) / F32(448.0)
            if use_ue8m0:
                m, e = np.frexp(s)
                s = F32(np.ldexp(1.0, e - 1 if m == 0.5 else e))
            assert sf[r, g].item() == s
            codes = e4m3.encode((seg * (F32(1.0) / s)).astype(np.float32))
            assert np.array_equal(codes, xq.view(torch.uint8).numpy()[r, g * 128 : g * 128 + seg.size])


def test_per_block_cast_ue8m0_vs_brute_force():
    """The use_ue8m0=True branch of per_block_cast_to_fp8_ref, as test_per_block_cast_vs_brute_force does for the
    other: scale = least power of two >= amax / 448 (frexp, not the oracle's bit test), codes from the bit-level
    encoder of the fp32 products."""
    g = torch.Generator().manual_seed(18)
    w = (0.02 * torch.randn(200, 300, generator=g) * torch.logspace(-2, 1, 300)).bfloat16()
    wq, ws = O.per_block_cast_to_fp8_ref(w, use_ue8m0=True)
    assert wq.shape == (200, 300) and ws.shape == (2, 3)
    wn = w.float().numpy()
    for bi in range(2):
        for bj in range(3):
            blk = wn[bi * 128 : (bi + 1) * 128, bj * 128 : (bj + 1) * 128]
            amax = max(F32(np.abs(blk).max()), F32(1e-4))
            s = F32(amax) / F32(448.0)
            m, e = np.frexp(s)
            s = F32(np.ldexp(1.0, e - 1 if m == 0.5 else e))
            assert ws[bi, bj].item() == s
            codes = e4m3.encode((blk * (F32(1.0) / s)).astype(np.float32))
            got = wq.view(torch.uint8).numpy()[bi * 128 : (bi + 1) * 128, bj * 128 : (bj + 1) * 128]
            assert np.array_equal(codes, got)


def test_ceil_log2_in_fp32_is_decided_by_the_bits_of_the_scale():
    """The device code of scale_ue8m0 evaluates no logarithm: for s = 2^n (1 + m 2^-23) it takes n + 1 unless
    m <= floor(ln 2 * 2^(j - 1)), j = floor(log2 |n|) (one less where n is minus a power of two; 0 for j < 2).  That
    closed form against the fp32 logarithm the oracle uses (torch) and against a float64 logarithm rounded to fp32, for
    every exponent the rule can meet and every mantissa near the thresholds, plus a random sample."""
    import numpy as np

    def closed_form(bits):
        n = (bits >> 23) - 127
        m = bits & 0x7FFFFF
        an = np.abs(n)
        j = np.where(an > 0, np.floor(np.log2(np.maximum(an, 1))).astype(np.int64), 0)
        j = j - ((n < 0) & ((an & (an - 1)) == 0)).astype(np.int64)
        keep = np.where((n != 0) & (j >= 2), np.floor(np.float32(0.69314718) * 2.0 ** (j - 1)).astype(np.int64), 0)
        return n + (m > keep)

    ns = np.arange(-34, 128)
    ms = np.concatenate([np.arange(0, 64), 2 ** np.arange(6, 23), np.array([0x7FFFFF, 0x7FFFFE, 0x400000])])
    bits = (((ns[:, None] + 127) << 23) | ms[None, :]).astype(np.int64).ravel()
    rng = np.random.default_rng(0)
    bits = np.concatenate([bits, ((rng.integers(93, 255, 200000) << 23) | rng.integers(0, 1 << 23, 200000)).astype(np.int64)])
    t = bits.astype(np.uint32).view(np.float32)
    via_f64 = np.ceil(np.log2(t.astype(np.float64)).astype(np.float32)).astype(np.int64)
    via_torch = torch.ceil(torch.log2(torch.from_numpy(t.copy()))).numpy().astype(np.int64)
    got = closed_form(bits)
    assert (got == via_f64).all() and (got == via_torch).all()
    # the rounding the rule is about does happen: some scales above 2^n keep n
    assert ((bits & 0x7FFFFF != 0) & (got == (bits >> 23) - 127)).any()
