"""The CPU oracle reproduces the committed golden vectors (guards against drift of
torch's RNG or cast behaviour between the container that wrote them and the host
that runs the tests)."""
import hashlib
import os

import numpy as np
import torch

from oracle import fp8_linear_oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _sha(t):
    return hashlib.sha256(t.contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()


def test_config1_golden():
    z = np.load(os.path.join(GOLD, "config1.npz"))
    r = O.run_config1(0)
    assert _sha(r["x"]) == str(z["x_sha"]) and _sha(r["w"]) == str(z["w_sha"])
    assert np.array_equal(r["xq"].view(torch.uint8).numpy(), z["xq"])
    assert np.array_equal(r["xs"].numpy().view(np.uint32), z["xs"].view(np.uint32))
    assert _sha(r["wq"]) == str(z["wq_sha"])
    assert np.array_equal(r["wq"].view(torch.uint8).numpy()[:8], z["wq_head"])
    assert np.array_equal(r["ws"].numpy().view(np.uint32), z["ws"].view(np.uint32))
    # fp32 matmul summation order may differ between hosts: within one bf16 step
    want = torch.from_numpy(z["c_bits"]).view(torch.bfloat16)
    torch.testing.assert_close(r["c"].float(), want.float(), rtol=2 ** -7, atol=2 ** -7)


def test_quant_variants_golden():
    z = np.load(os.path.join(GOLD, "quant_variants.npz"))
    x, _ = O.make_config1(0)
    for name, fn in [
        ("group", lambda t: O.per_token_group_quant_fp8_ref(t, 128)),
        ("group_ue8m0", lambda t: O.per_token_group_quant_fp8_ref(t, 128, scale_ue8m0=True)),
        ("act_ue8m0", lambda t: O.act_quant_ref(t, 128, "ue8m0")),
        ("div", lambda t: O.per_token_group_quant_fp8_div_ref(t, 128)),
    ]:
        q, s = fn(x)
        assert np.array_equal(q.view(torch.uint8).numpy(), z[name + "_q"]), name
        assert np.array_equal(s.numpy().view(np.uint32), z[name + "_s"].view(np.uint32)), name


def test_scaled_mm_golden():
    z = np.load(os.path.join(GOLD, "scaled_mm.npz"))
    a = torch.from_numpy(z["a"]).view(torch.float8_e4m3fn)
    b = torch.from_numpy(z["b_t"]).view(torch.float8_e4m3fn).t()
    bias = torch.from_numpy(z["bias_bits"]).view(torch.bfloat16)
    out = O.scaled_mm_ref(a, b, torch.from_numpy(z["sa"]), torch.from_numpy(z["sb"]), torch.bfloat16, bias)
    # fp32 mm summation order may differ between hosts: compare in value, tightly
    want = torch.from_numpy(z["out_bits"]).view(torch.bfloat16)
    torch.testing.assert_close(out.float(), want.float(), rtol=2 ** -7, atol=2 ** -7)
