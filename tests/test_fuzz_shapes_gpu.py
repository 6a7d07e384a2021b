"""Seeded random shapes through the GEMM entry points, every element checked on the device.

The launch planner chooses kernel, tile height, K cuts and tail launches from (M, N, K); the tuned shapes of the
benchmark exercise a few dozen of its branches.  These walks draw shapes off that grid -- ragged N, K that is
not a multiple of 128 for the row/column modes, batches, every row-count regime -- with a fixed seed, name each case
on stdout before it is launched (so a fault names its shape) and stop at the first mismatch.

The comparison is with torch's own fp32 GEMM of the dequantised operands on the device: a cross-check by an
independent implementation, not the oracle (the oracle comparisons are in the other test files).  Operands are
N(0, 1) codes with scales in [0.25, 1.25), so results are O(sqrt(K)) ~ 10 .. 100 and the absolute part of the bar is
scaled with them: |got - want| <= 1e-2 |want| + 2.5e-3 max|want| + 1e-3 for the block-scaled calls (1.6e-2 |want| for
the row/column calls, whose bias is added after a first rounding to the 16-bit output type, as the reference's
epilogue does: src/flag_gems/fused/cutlass_scaled_mm.py:288-305)."""
import random

import pytest
import torch

import flag_gems

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn


def _block_reference(x, xs, w, ws):
    xd = x.float() * xs.repeat_interleave(128, dim=-1)[..., : x.shape[-1]]
    wsd = ws.repeat_interleave(128, dim=-2)[..., : w.shape[-2], :].repeat_interleave(128, dim=-1)[..., : w.shape[-1]]
    return xd @ (w.float() * wsd).transpose(-1, -2)


def test_block_scaled_shapes_walk():
    rng = random.Random(20240607)
    torch.manual_seed(0)
    for it in range(120):
        kind = rng.choice(["dense", "dense", "batch"])
        K = 128 * rng.randint(1, 40)
        if kind == "dense":
            M = rng.choice([rng.randint(1, 64), rng.randint(33, 64), rng.randint(65, 300), rng.randint(129, 1400),
                            256 * rng.randint(1, 6), 256 * rng.randint(7, 18)])
            N = rng.choice([128 * rng.randint(1, 64), 8 * rng.randint(1, 900), 256 * rng.randint(1, 40), 28672, 24576])
            tag = f"case {it}: dense M={M} N={N} K={K}"
            print(tag, flush=True)
            x = torch.randn(M, K, device=DEV).to(FP8)
            xs = torch.rand(M, K // 128, device=DEV) + 0.25
            w = torch.randn(N, K, device=DEV).to(FP8)
            ws = torch.rand((N + 127) // 128, K // 128, device=DEV) + 0.25
            got = flag_gems.w8a8_block_fp8_matmul(x, w, xs, ws, [128, 128])
        else:
            B = rng.randint(2, 20)
            M = rng.choice([rng.randint(1, 32), rng.randint(33, 64), rng.randint(65, 128), rng.randint(129, 520)])
            N = 128 * rng.randint(1, 12)
            tag = f"case {it}: batch B={B} M={M} N={N} K={K}"
            print(tag, flush=True)
            x = torch.randn(B, M, K, device=DEV).to(FP8)
            xs = torch.rand(B, M, K // 128, device=DEV) + 0.25
            w = torch.randn(B, N, K, device=DEV).to(FP8)
            ws = torch.rand(B, N // 128, K // 128, device=DEV) + 0.25
            got = flag_gems.w8a8_block_fp8_bmm(x, w, xs, ws, [128, 128])
        want = _block_reference(x, xs, w, ws)
        assert torch.isfinite(got.float()).all(), tag
        err = (got.float() - want).abs()
        tol = 1e-2 * want.abs() + 2.5e-3 * want.abs().max().item() + 1e-3
        n_bad = int((err > tol).sum())
        assert n_bad == 0, f"{tag}: {n_bad} elements outside the bar, max error {err.max().item():.4g}"


def test_row_column_scaled_shapes_walk():
    rng = random.Random(977)
    torch.manual_seed(1)
    for it in range(80):
        i8 = rng.random() < 0.4
        K = 16 * rng.randint(1, 300) if rng.random() < 0.3 else 128 * rng.randint(1, 48)
        M = rng.choice([rng.randint(1, 64), rng.randint(33, 64), rng.randint(65, 300), rng.randint(129, 1400), 256 * rng.randint(1, 8)])
        N = rng.choice([16 * rng.randint(1, 500), 256 * rng.randint(1, 40), 28672, 24576, 8192])
        odt = rng.choice([torch.bfloat16, torch.float16])
        one_a, one_b, with_bias = rng.random() < 0.3, rng.random() < 0.3, rng.random() < 0.6
        tag = (f"case {it}: {'int8' if i8 else 'fp8'} M={M} N={N} K={K} {odt} bias={with_bias} "
               f"scale_a={'scalar' if one_a else 'rows'} scale_b={'scalar' if one_b else 'columns'}")
        print(tag, flush=True)
        if i8:
            a = torch.randint(-127, 128, (M, K), device=DEV, dtype=torch.int8)
            b = torch.randint(-127, 128, (N, K), device=DEV, dtype=torch.int8)
            sa = torch.rand(M, 1, device=DEV) * 1e-2 + 1e-3
            sb = torch.rand(N, 1, device=DEV) * 1e-2 + 1e-3
        else:
            a = torch.randn(M, K, device=DEV).to(FP8)
            b = torch.randn(N, K, device=DEV).to(FP8)
            sa = torch.rand(M, 1, device=DEV) + 0.25
            sb = torch.rand(N, 1, device=DEV) + 0.25
        if one_a:
            sa = sa[:1].contiguous()
        if one_b:
            sb = sb[:1].contiguous()
        bias = (torch.randn(N, device=DEV) * 5).to(odt) if with_bias else None
        c = torch.empty(M, N, device=DEV, dtype=odt)
        flag_gems.cutlass_scaled_mm(c, a, b.t(), sa, sb, bias)
        want = (a.float() @ b.float().t()) * sa * sb.reshape(1, -1)
        if bias is not None:
            want = want.to(odt).float() + bias.float()
        assert torch.isfinite(c.float()).all(), tag
        err = (c.float() - want).abs()
        tol = 1.6e-2 * want.abs() + 2.5e-3 * want.abs().max().item() + 1e-3
        n_bad = int((err > tol).sum())
        assert n_bad == 0, f"{tag}: {n_bad} elements outside the bar, max error {err.max().item():.4g}"


def test_grouped_shapes_walk():
    """Grouped (expert) products with random segment tables: 1 .. 16 experts, empty and one-row segments, few rows per
    segment (64- and 128-row tiles) up to thousands (256-row tiles, more tiles than compute units, the last round cut
    along K), rows gathered through an index, results scattered and weighted, bf16 and fp16 -- every element against
    torch's fp32 GEMM of the dequantised operands, segment by segment."""
    rng = random.Random(4711)
    torch.manual_seed(2)
    for it in range(60):
        E = rng.choice([1, 2, 3, 8, 16])
        K = 128 * rng.choice([1, 4, 8, 16, 24, 32, 56, 64])
        N = rng.choice([128 * rng.randint(1, 32), 8 * rng.randint(16, 500), 256 * rng.randint(1, 16)])
        avg = rng.choice([3, 20, 60, 100, 200, 700, 2500])
        counts = [max(0, int(rng.gauss(avg, avg / 2))) if rng.random() > 0.15 else rng.choice([0, 1]) for _ in range(E)]
        if sum(counts) == 0:
            counts[0] = 5
        while sum(counts) * (N + K) > 3.0e8:  # keep a case under a few hundred MB
            counts = [c // 2 for c in counts]
        M = sum(counts)
        ends = torch.tensor([sum(counts[: i + 1]) for i in range(E)], dtype=torch.int32, device=DEV)
        mode = rng.choice(["sorted", "gather", "scatter", "scatter+weights"])
        odt = rng.choice([torch.bfloat16, torch.float16])
        top_k = rng.choice([1, 2, 4]) if mode != "sorted" else 1
        tag = f"case {it}: grouped E={E} rows={counts} N={N} K={K} {mode} top_k={top_k} {odt}"
        print(tag, flush=True)
        w = torch.randn(E, N, K, device=DEV).to(FP8)
        ws = torch.rand(E, (N + 127) // 128, K // 128, device=DEV) + 0.25
        if mode == "sorted":
            x = torch.randn(M, K, device=DEV).to(FP8)
            xs = torch.rand(M, K // 128, device=DEV) + 0.25
            got = flag_gems.grouped_w8a8_block_fp8_matmul(x, w, xs, ws, ends, [128, 128], odt)
            x_rows, xs_rows, out_rows, wts = x, xs, None, None
        else:
            T = (M + top_k - 1) // top_k  # tokens; slot s reads token s // top_k
            x = torch.randn(T, K, device=DEV).to(FP8)
            xs = torch.rand(T, K // 128, device=DEV) + 0.25
            slots = torch.randperm(T * top_k, device=DEV)[:M].to(torch.int32)  # sorted row m is slot slots[m]
            src = (slots.long() // top_k)
            x_rows, xs_rows = x[src], xs[src]
            kw = dict(row_index=slots, index_divisor=top_k)
            out_rows, wts = None, None
            if mode != "gather":
                kw["scatter_rows"] = T * top_k
                out_rows = slots.long()
                if mode == "scatter+weights":
                    wts = torch.rand(T * top_k, device=DEV) + 0.5
                    kw["row_weights"] = wts
            got = flag_gems.grouped_w8a8_block_fp8_matmul(x, w, xs, ws, ends, [128, 128], odt, **kw)
        begin = 0
        for e in range(E):
            end = int(ends[e])
            if end > begin:
                want = _block_reference(x_rows[begin:end], xs_rows[begin:end], w[e], ws[e])
                if out_rows is None:
                    mine = got[begin:end].float()
                else:
                    mine = got[out_rows[begin:end]].float()
                    if wts is not None:
                        want = want * wts[out_rows[begin:end]][:, None]
                assert torch.isfinite(mine).all(), tag
                err = (mine - want).abs()
                tol = 1e-2 * want.abs() + 2.5e-3 * want.abs().max().item() + 1e-3
                n_bad = int((err > tol).sum())
                assert n_bad == 0, f"{tag}: expert {e}: {n_bad} elements outside the bar, max error {err.max().item():.4g}"
            begin = end
