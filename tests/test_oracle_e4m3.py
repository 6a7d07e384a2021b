"""Pins oracle/e4m3.py and torch's e4m3fn cast against each other and against the
format definition."""
import math

import numpy as np
import torch

from oracle import e4m3


def test_decode_table_known_values():
    t = e4m3.decode_table()
    assert t[0x00] == 0.0 and t[0x80] == 0.0 and math.copysign(1, t[0x80]) == -1
    assert t[0x01] == 2.0 ** -9  # smallest subnormal
    assert t[0x07] == 7 * 2.0 ** -9  # largest subnormal
    assert t[0x08] == 2.0 ** -6  # smallest normal
    assert t[0x38] == 1.0
    assert t[0x7E] == 448.0 and t[0xFE] == -448.0
    assert math.isnan(t[0x7F]) and math.isnan(t[0xFF])
    # strictly increasing over the positive finite codes
    assert np.all(np.diff(t[:0x7F]) > 0)


def test_decode_table_matches_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float().numpy()
    mine = e4m3.decode_table()
    assert np.array_equal(np.isnan(ref), np.isnan(mine))
    ok = ~np.isnan(ref)
    assert np.array_equal(ref[ok], mine[ok])
    assert np.array_equal(np.signbit(ref[ok]), np.signbit(mine[ok]))


def test_encode_all_bf16_patterns_matches_torch():
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16).float()
    ref = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    mine = e4m3.encode(x.numpy())
    assert np.array_equal(ref, mine)


def test_encode_random_fp32_and_midpoints_matches_torch():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1 << 18, generator=g) * torch.exp(4 * torch.randn(1 << 18, generator=g))
    t = torch.from_numpy(e4m3.decode_table()[:0x7F].copy())
    mid = (t[1:] + t[:-1]) / 2  # exact in fp32
    eps = torch.tensor([0.0, 1e-7, -1e-7])
    mids = (mid[:, None] * (1 + eps[None, :])).flatten()
    x = torch.cat([x, mids, -mids, torch.tensor([464.0, 465.0, 463.99, 1e9, -1e9, float("inf"), float("-inf")])])
    ref = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    mine = e4m3.encode(x.numpy())
    assert np.array_equal(ref, mine)


def test_encode_against_nearest_value_search():
    g = np.random.default_rng(2)
    vals = np.concatenate(
        [
            g.standard_normal(300).astype(np.float32) * 100,
            g.standard_normal(300).astype(np.float32) * 0.01,
            np.array([0.3, 448, 464, 465, 500, -17.3, 1e-4, 2.0 ** -10, 3 * 2.0 ** -10, 0.0, -0.0], dtype=np.float32),
        ]
    )
    mine = e4m3.encode(vals)
    for v, c in zip(vals, mine):
        assert int(c) == e4m3.encode_scalar_reference(float(v)), v


def test_known_answers():
    # observed torch 2.10 CPU behaviour, stated as literal codes
    x = np.array([0.3, 448.0, 464.0, 465.0, 500.0, -17.3, 1e-4, 2.0 ** -10, float("nan"), -float("nan"), float("inf")], dtype=np.float32)
    want = [0x2A, 0x7E, 0x7E, 0x7F, 0x7F, 0xD9, 0x00, 0x00, 0x7F, 0xFF, 0x7F]
    assert list(e4m3.encode(x)) == want
    assert list(torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()) == want
