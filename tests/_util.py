"""Helpers shared by the GPU parity tests."""
import torch


def codes(t: torch.Tensor) -> torch.Tensor:
    """fp8 tensor -> uint8 codes on CPU with NaN codes folded to 0x7F (the sign of a NaN that an
    invalid operation produces differs between x86 hosts and the GPU; both are NaN)."""
    c = t.detach().cpu().contiguous().view(torch.uint8).clone()
    c[(c & 0x7F) == 0x7F] = 0x7F
    return c


def bits32(t: torch.Tensor) -> torch.Tensor:
    b = t.detach().cpu().contiguous().view(torch.int32).clone()
    nan = (b & 0x7FFFFFFF) > 0x7F800000
    b[nan] = 0x7FC00000
    return b


def assert_codes_equal(got, want, what=""):
    g, w = codes(got), codes(want)
    if not torch.equal(g, w):
        bad = (g != w).nonzero()
        raise AssertionError(f"{what}: {bad.shape[0]} of {g.numel()} codes differ, first at {bad[0].tolist()}: "
                             f"got {g[tuple(bad[0])].item():#x} want {w[tuple(bad[0])].item():#x}")


def assert_scales_equal(got, want, what=""):
    g, w = bits32(got), bits32(want)
    if not torch.equal(g, w):
        bad = (g != w).nonzero()
        i = tuple(bad[0])
        raise AssertionError(f"{what}: {bad.shape[0]} of {g.numel()} scales differ, first at {bad[0].tolist()}: "
                             f"got {got.detach().cpu()[i].item()!r} want {want.detach().cpu()[i].item()!r}")
