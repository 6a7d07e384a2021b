"""The launch planner picks a kernel from (M, N, K) by thresholds that were fitted on the benchmark shapes.  This test
walks shapes off that grid (decode-sized M and wide weights included) and checks that none falls into a slow corner: every call must finish within twice a
deliberately loose cost model (the slower of 1.2 PFLOP/s and 2.5 TB/s, plus 15 us of fixed cost -- about half of what
the tuned shapes reach), so a rule that sends a shape to a kernel three times too slow for it fails here.  Results
are checked elsewhere; this file only times.

A wall-clock figure is no correctness signal, and a loaded or clock-throttled box can miss a limit with no change to the
code: a miss is therefore reported as a warning with the table of slow shapes (pytest's warnings summary shows it), and
the tests fail only for a call more than eight times over the model, which no throttling explains."""
import warnings

import pytest
import torch

import flag_gems

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn

NK = [(1000, 1024), (2112, 7168), (3000, 3072), (5120, 2048), (7168, 2304), (12288, 1536), (4096, 8192), (1536, 16384),
      (28672, 4096), (512, 4096), (512, 7168), (2048, 16384), (32768, 1024), (65536, 2048), (20480, 8192)]
MS = [1, 3, 9, 17, 33, 48, 65, 100, 130, 200, 300, 400, 600, 777, 1000, 1100, 1500, 2048, 3000, 5000]


def _model_us(M, N, K):
    flops = 2.0 * M * N * K
    nbytes = M * K + N * K + 2.0 * M * N + 4.0 * (M + N / 128) * (K / 128)
    return max(flops / 1.2e15, nbytes / 2.5e12) * 1e6 + 15.0


def _report(slow, columns):
    """Warn about calls over their limit; fail only for one that is more than four limits (eight models) over."""
    if not slow:
        return
    warnings.warn(f"slower than twice the cost model {columns}: {slow}")
    far = [row for row in slow if row[-2] > 4.0 * row[-1]]
    assert not far, f"far off the cost model {columns}: {far}"


def _time_us(fn):
    fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(3):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(5):
            fn()
        end.record()
        end.synchronize()
        best = min(best, start.elapsed_time(end) * 1e3 / 5)
    return best


@pytest.mark.parametrize("N,K", NK)
def test_no_shape_is_far_off_the_cost_model(N, K):
    g = torch.Generator(device=DEV).manual_seed(N + K)
    w = torch.randn(N, K, device=DEV, generator=g).to(FP8)
    ws = torch.rand((N + 127) // 128, K // 128, device=DEV, generator=g) + 0.5
    slow = []
    for M in MS:
        x = torch.randn(M, K, device=DEV, generator=g).to(FP8)
        xs = torch.rand(M, K // 128, device=DEV, generator=g) + 0.5
        us = _time_us(lambda: flag_gems.w8a8_block_fp8_matmul(x, w, xs, ws, [128, 128]))
        # eager launches from Python cost ~15-20 us of host time each: short kernels are bound by that, not by the GPU
        limit = 2.0 * _model_us(M, N, K) + 20.0
        if us > limit:
            slow.append((M, N, K, round(us, 1), round(limit, 1)))
    _report(slow, "(M, N, K, measured us, limit us)")


@pytest.mark.parametrize("N,K", [(7168, 2304), (4096, 8192), (2112, 7168)])
def test_output_types_and_scale_modes_stay_within_the_same_model(N, K):
    """The same walk for fp16 and fp32 results and for the row/column scaled entry point (fp8 and int8 operands): a
    result type or a scale mode that only a slower kernel serves shows up here (the persistent kernel used to write
    bf16 only, and fp16 results above 128 rows took six times as long in the row/column mode)."""
    g = torch.Generator(device=DEV).manual_seed(N * K)
    w = torch.randn(N, K, device=DEV, generator=g).to(FP8)
    ws = torch.rand((N + 127) // 128, K // 128, device=DEV, generator=g) + 0.5
    wi = torch.randint(-128, 128, (N, K), device=DEV, generator=g, dtype=torch.int32).to(torch.int8)
    sb = torch.rand(1, N, device=DEV, generator=g) + 0.5
    slow = []
    for M in (1, 17, 48, 100, 200, 600, 1500, 4096):
        x = torch.randn(M, K, device=DEV, generator=g).to(FP8)
        xi = torch.randint(-128, 128, (M, K), device=DEV, generator=g, dtype=torch.int32).to(torch.int8)
        xs = torch.rand(M, K // 128, device=DEV, generator=g) + 0.5
        sa = torch.rand(M, 1, device=DEV, generator=g) + 0.5
        for dt in (torch.float16, torch.float32, torch.bfloat16):
            c = torch.empty(M, N, dtype=dt, device=DEV)
            calls = {"row/column fp8": lambda: flag_gems.cutlass_scaled_mm(c, x, w.t(), sa, sb, None),
                     "row/column int8": lambda: flag_gems.cutlass_scaled_mm(c, xi, wi.t(), sa, sb, None)}
            if dt != torch.bfloat16:  # (bf16 block-scaled: the test above)
                calls["block"] = lambda: flag_gems.w8a8_block_fp8_matmul(x, w, xs, ws, [128, 128], output_dtype=dt)
            for name, fn in calls.items():
                us = _time_us(fn)
                # fp32 results are twice the bytes; the model counts two per element
                limit = 2.0 * _model_us(M, N, K) + 20.0 + (2.0 * M * N / 2.5e12 * 1e6 if dt == torch.float32 else 0.0)
                if us > limit:
                    slow.append((name, str(dt), M, N, K, round(us, 1), round(limit, 1)))
    _report(slow, "(call, type, M, N, K, measured us, limit us)")
