"""Writes the committed golden vectors under tests/golden/ from the CPU oracle.

    python tests/golden/make_golden.py

The reference keeps no stored vectors for this path (its tests recompute a torch
reference from a seed at run time), so these are produced by the restated oracle,
whose functions are pinned by tests/test_oracle_*.py.  Inputs are regenerated
from the seed by ``oracle.fp8_linear_oracle.make_config1``; only outputs (and
SHA-256 digests of the inputs, to catch RNG drift) are stored.
"""
import hashlib
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import fp8_linear_oracle as O  # noqa: E402


def sha(t: torch.Tensor) -> str:
    return hashlib.sha256(t.contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()


def main():
    r = O.run_config1(0)
    np.savez_compressed(
        os.path.join(HERE, "config1.npz"),
        x_sha=np.array(sha(r["x"])),
        w_sha=np.array(sha(r["w"])),
        xq=r["xq"].view(torch.uint8).numpy(),
        xs=r["xs"].numpy(),
        wq_sha=np.array(sha(r["wq"])),
        wq_head=r["wq"].view(torch.uint8).numpy()[:8],
        ws=r["ws"].numpy(),
        c_bits=r["c"].view(torch.int16).numpy(),
    )
    # group quantizer (division quotient) and ue8m0 act_quant on the same X
    x = r["x"]
    gq, gs = O.per_token_group_quant_fp8_ref(x, 128)
    gq8, gs8 = O.per_token_group_quant_fp8_ref(x, 128, scale_ue8m0=True)
    aq8, as8 = O.act_quant_ref(x, 128, "ue8m0")
    dq, ds = O.per_token_group_quant_fp8_div_ref(x, 128)
    np.savez_compressed(
        os.path.join(HERE, "quant_variants.npz"),
        group_q=gq.view(torch.uint8).numpy(), group_s=gs.numpy(),
        group_ue8m0_q=gq8.view(torch.uint8).numpy(), group_ue8m0_s=gs8.numpy(),
        act_ue8m0_q=aq8.view(torch.uint8).numpy(), act_ue8m0_s=as8.numpy(),
        div_q=dq.view(torch.uint8).numpy(), div_s=ds.numpy(),
    )
    # scaled_mm: per-token x per-channel with bias, small
    g = torch.Generator().manual_seed(0)
    a32 = torch.randn(32, 256, generator=g)
    b32 = torch.randn(256, 64, generator=g)
    bias = torch.randn(64, generator=g).bfloat16()
    sa = a32.abs().amax(1, keepdim=True) / 448.0
    sb = b32.abs().amax(0, keepdim=True) / 448.0
    a = (a32 / sa).to(torch.float8_e4m3fn)
    b = (b32 / sb).t().contiguous().t().to(torch.float8_e4m3fn)
    out = O.scaled_mm_ref(a, b, sa, sb, torch.bfloat16, bias)
    np.savez_compressed(
        os.path.join(HERE, "scaled_mm.npz"),
        a=a.view(torch.uint8).numpy(), b_t=b.t().contiguous().view(torch.uint8).numpy(),
        sa=sa.numpy(), sb=sb.numpy(), bias_bits=bias.view(torch.int16).numpy(),
        out_bits=out.view(torch.int16).numpy(),
    )
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
