"""GPU parity of the 128 x 128 weight quantizer against the CPU oracle: bit-exact codes and scales.

The oracle function restates the torch helper the reference builds its block-quantized weights with
(tests/test_fp8_einsum.py:89-103 of the reference); everything goes through the C ABI via
flag_gems.per_block_cast_to_fp8."""
import hashlib
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


def _w(shape, seed, dtype=torch.bfloat16, kind="weights"):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(*shape, generator=g)
    if kind == "weights":
        w = 0.02 * w
    elif kind == "wide":
        w = w * torch.exp(3 * torch.randn(*shape, generator=g))
    return w.to(dtype)


def _check(x, ue8m0, what=""):
    want_q, want_s = O.per_block_cast_to_fp8_ref(x, use_ue8m0=ue8m0)
    q, s = flag_gems.per_block_cast_to_fp8(x.to(DEV), use_ue8m0=ue8m0)
    assert q.dtype == torch.float8_e4m3fn and q.shape == x.shape and q.is_contiguous()
    assert s.dtype == torch.float32 and s.shape == want_s.shape
    assert_scales_equal(s, want_s, what)
    assert_codes_equal(q, want_q, what)


@pytest.mark.parametrize("shape", [(512, 1024), (2112, 7168), (128, 128), (300, 200), (129, 8), (1, 5), (1000, 515),
                                   (4096, 14336)])
@pytest.mark.parametrize("ue8m0", [False, True])
def test_block_quant_matches_oracle(shape, ue8m0):
    _check(_w(shape, 0), ue8m0, f"{shape}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("kind", ["weights", "wide"])
def test_block_quant_dtypes_and_ranges(dtype, kind):
    if dtype == torch.float16 and kind == "wide":
        pytest.skip("the wide distribution overflows float16")
    for ue8m0 in (False, True):
        _check(_w((384, 640), 1, dtype, kind), ue8m0, f"{dtype} {kind}")
        _check(_w((130, 257), 2, dtype, kind), ue8m0, f"{dtype} {kind} ragged")


def test_block_quant_strided_and_unaligned_rows():
    big = _w((400, 1100), 3).to(DEV)
    for view in (big[:, :1024], big[16:272, 8:520], big[:, 1:1025], big[3:, 5:900]):
        want_q, want_s = O.per_block_cast_to_fp8_ref(view.cpu().contiguous(), use_ue8m0=False)
        q, s = flag_gems.per_block_cast_to_fp8(view, use_ue8m0=False)
        assert_scales_equal(s, want_s)
        assert_codes_equal(q, want_q)
    # a transposed view is copied to unit column stride first
    t = big.t()
    want_q, want_s = O.per_block_cast_to_fp8_ref(t.cpu().contiguous(), use_ue8m0=True)
    q, s = flag_gems.per_block_cast_to_fp8(t, use_ue8m0=True)
    assert_scales_equal(s, want_s)
    assert_codes_equal(q, want_q)


def test_block_quant_special_values():
    x = _w((384, 384), 4, kind="randn")
    x[:128, :128] = 0.0                  # all-zero block: scale comes from the floor
    x[130, 5] = float("nan")             # NaN poisons its block
    x[10, 140] = float("inf")            # Inf: scale inf, finite elements -> 0, Inf -> NaN
    x[200, 200] = -3e38                  # lone huge element
    x[256:, 256:] = 2.0 ** -130          # below the bf16 normal range: the floor decides
    x[300, 10] = float("-inf")
    for ue8m0 in (False, True):
        _check(x, ue8m0, f"special ue8m0={ue8m0}")


def test_block_quant_golden_weights():
    z = np.load(os.path.join(GOLD, "config1.npz"))
    _, w = O.make_config1(0)
    q, s = flag_gems.per_block_cast_to_fp8(w.to(DEV), use_ue8m0=False)
    codes = q.cpu().view(torch.uint8).numpy()
    assert hashlib.sha256(codes.tobytes()).hexdigest() == str(z["wq_sha"])
    assert np.array_equal(codes[:8], z["wq_head"])
    assert np.array_equal(s.cpu().numpy().view(np.uint32), z["ws"].view(np.uint32))


def test_block_quant_feeds_the_gemm():
    """Quantize activations and weights on the device, multiply, compare with the oracle's whole path."""
    want = O.run_config1(0)
    xq, xs = flag_gems.act_quant_triton(want["x"].to(DEV), 128)
    wq, ws = flag_gems.per_block_cast_to_fp8(want["w"].to(DEV), use_ue8m0=False)
    c = flag_gems.w8a8_block_fp8_matmul(xq, wq, xs, ws, [128, 128])
    torch.testing.assert_close(c.cpu().float(), want["c"].float(), rtol=1e-2, atol=1e-2)


def test_block_quant_full_size_properties():
    """Largest weight of the benchmark configurations (28672 x 4096): every block's largest code is +-448 (or the
    block is below the floor), and dequantised values are within half a code step of the input."""
    torch.manual_seed(0)
    w = (0.02 * torch.randn(28672, 4096, device=DEV)).bfloat16()
    q, s = flag_gems.per_block_cast_to_fp8(w, use_ue8m0=False)
    blk = q.float().view(224, 128, 32, 128).abs().amax(dim=(1, 3))
    assert torch.all(blk == 448.0)
    deq = q.float().view(224, 128, 32, 128) * s.view(224, 1, 32, 1)
    err = (deq - w.float().view(224, 128, 32, 128)).abs()
    assert float((err / (s.view(224, 1, 32, 1) * 448.0)).max()) <= 2.0 ** -4 + 1e-6  # half of the coarsest e4m3 step
    with pytest.raises(NotImplementedError):
        flag_gems.per_block_cast_to_fp8(w[:256, :256], gran_k=64)


def test_block_quant_empty():
    q, s = flag_gems.per_block_cast_to_fp8(torch.empty(0, 256, dtype=torch.bfloat16, device=DEV))
    assert q.shape == (0, 256) and s.shape == (0, 2)
