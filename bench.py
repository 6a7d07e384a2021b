#!/usr/bin/env python3
"""Benchmark of the FP8 quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = SWEEPS_PER_STEP (16) passes over the DeepSeek-V3 block-fp8 GEMM sweep that the headline metric is quoted on
(a single pass takes about 2 ms, so 20 steps of one pass would be a 40 ms timed region):
M in {1, 8, 64, 512, 2048, 4096} x (N, K) in {(2112,7168), (24576,1536), (32768,512), (7168,16384),
(4608,7168), (7168,2304)}, e4m3fn operands already resident in HBM (1x128 activation scales,
128x128 weight scales, bf16 output).  `value` is the sweep's total 2*M*N*K divided by the wall
time of the timed steps.  For M <= 64 every call uses a different copy of the weights out of a pool
larger than the 256 MB Infinity Cache, so small-M numbers are HBM numbers, not cache numbers.

Prints ONE JSON line with the driver's fields plus
  roofline      dominant kernel (the M = 4096 GEMMs): achieved TFLOP/s from HIP-event timings, against
                the dense FP8 MFMA peak
  cpu_baseline  the CPU oracle (torch restatement of the reference's torch implementation) timed on
                the host cores on a bounded sample of the same sweep
  detail        per-(M, N, K) time, TFLOP/s, GB/s and roofline fractions (MFMA for M >= 512, HBM below)
  block_fp8_gemm_pow2_scales_m4096, cutlass_scaled_mm_n8192_k8192_bias, cutlass_scaled_mm_int8_n8192_k8192_bias,
  llama3_8b_linears
                the other configurations of the path (per-token x per-channel scaled GEMM with bias, fp8 and int8
                operands; Llama-3-8B
                linears as GEMM alone and as act_quant + GEMM), graph replays of one shape at a time with ONE copy
                of the weights (small-M figures there may be served by the 256 MB Infinity Cache), not part of `value`
  rows_at_the_hand_over_points
                the block GEMM at the row counts where one kernel hands over to the next (16 | 17, 32 | 33, 64 | 65,
                128 | 129) on three weights, weights rotated through 512 MB; not part of `value`
  mixtral_moe_grouped_gemm
                Mixtral-8x7B expert layers: 8 experts, top-2 over T tokens with Zipf(1.1) expert loads, rows sorted by
                expert; the grouped block-fp8 GEMM with W1 [8,28672,4096] and W2 [8,4096,14336]; not part of `value`
  mixtral_moe_layer
                the whole expert layer on those weights (fused_experts_impl: quantize, GEMM 1 with gathered rows,
                SiLU-and-mul + quantize, GEMM 2 with scattered weighted rows, sum over the slots), end to end
  eager_host_overhead
                host time per eager call (no graph) of fp8_matmul, of its allocation-only twin fp8_matmul_noop and of the
                bare C-ABI call, at M = 1 on the smallest and the largest weight, next to the kernel's time
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0  # MI355X dense FP8 MFMA, published
PEAK_HBM_GBPS = 8000.0    # MI355X HBM3E, published
DSV3_NK = [(2112, 7168), (24576, 1536), (32768, 512), (7168, 16384), (4608, 7168), (7168, 2304)]
DSV3_M = [1, 8, 64, 512, 2048, 4096]
DETAIL_M = [1, 8, 16, 64, 512, 2048, 4096]  # per-shape timings also cover M = 16 (decode bar: M <= 16)
CACHE_BYTES = 512 << 20   # rotate small-M weights through at least this much memory
SWEEPS_PER_STEP = 16      # passes over the 36-GEMM sweep in one step
LAUNCHES = 100            # back-to-back launches per timed graph replay
REPEATS = 6               # timed replays per shape; the first is dropped, the median of the other five is reported

# Bytes that crossed the L2 <-> memory-fabric boundary in one M = 4096 call (the persistent kernel and, where the
# call makes one, the transposition of the activation scales before it), from two
# hardware-counter runs of `bench.py --counter-pass` (FETCH_SIZE, then WRITE_SIZE, in KiB per dispatch), each
# scaled by what the same counter read for the 256 MiB device copy issued first in that run (FETCH_SIZE read
# half of the copied bytes, factor 2.0; WRITE_SIZE read all of them, factor 1.0).  (N, K) -> (fetch, write) KiB.
TRAFFIC_M4096_KIB = {
    (2112, 7168): (2.0 * 63360.5, 17792.0),
    (24576, 1536): (2.0 * 112156.3, 196800.0),
    (32768, 512): (2.0 * 48261.2, 262144.0),
    (7168, 16384): (2.0 * 366004.8, 59392.0),
    (4608, 7168): (2.0 * 123769.4, 70568.0),
    (7168, 2304): (2.0 * 51600.6, 57632.0),
}


def gemm_flops(m, n, k):
    return 2.0 * m * n * k


def gemm_bytes(m, n, k):
    kb, nb = (k + 127) // 128, (n + 127) // 128
    return m * k + n * k + 4 * m * kb + 4 * nb * kb + 2 * m * n


def moe_row_ends(tokens, experts, top_k, seed):
    """Cumulative int32 row ends of tokens * top_k rows sorted by expert; expert loads follow a Zipf(1.1) law over a
    seeded permutation of the experts."""
    import torch

    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(experts, generator=g)
    p = torch.zeros(experts, dtype=torch.float64)
    p[perm] = 1.0 / torch.arange(1, experts + 1, dtype=torch.float64) ** 1.1
    ids = torch.multinomial(p / p.sum(), tokens * top_k, replacement=True, generator=g)
    return torch.cumsum(torch.bincount(ids, minlength=experts), 0).to(torch.int32)


def make_weight(n, k, gen, dev):
    """W ~ N(0, 0.02) quantized per 128x128 block on the device with torch ops (data preparation)."""
    import torch

    w = torch.randn(n, k, device=dev, generator=gen) * 0.02
    np_, kp = (n + 127) // 128 * 128, (k + 127) // 128 * 128
    wp = torch.zeros(np_, kp, device=dev)
    wp[:n, :k] = w
    blk = wp.view(np_ // 128, 128, kp // 128, 128)
    amax = blk.abs().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    sf = amax / 448.0
    q = (blk * (1.0 / sf)).to(torch.float8_e4m3fn).view(np_, kp)[:n, :k].contiguous()
    return q, sf.view(np_ // 128, kp // 128).contiguous()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--counter-pass", action="store_true",
                    help="for hardware-counter runs: one 256 MiB device copy (calibration), then one eager launch of "
                         "every (M, N, K) of the per-shape table, an elementwise marker kernel before each, and one "
                         "quantizer launch; no timing, no JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; run with --gpus 1 "
              "(the path shards by N or K across GPUs with no change to the kernels)", file=sys.stderr)
        sys.exit(2)

    import torch

    import flag_gems

    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(0)

    # ---- synthetic inputs, resident in HBM
    acts = {}     # (M, K) -> (xq, xs)
    weights = {}  # (N, K) -> list of (wq, ws) copies
    for (n, k) in DSV3_NK:
        wq, ws = make_weight(n, k, gen, dev)
        copies = max(1, -(-CACHE_BYTES // (n * k)))
        pool = [(wq, ws)] + [(wq.clone(), ws.clone()) for _ in range(copies - 1)]
        weights[(n, k)] = pool
        for m in DETAIL_M:
            if (m, k) not in acts:
                x = torch.randn(m, k, device=dev, generator=gen).bfloat16()
                acts[(m, k)] = flag_gems.act_quant_triton(x, 128)
    torch.cuda.synchronize()

    calls = [(m, n, k) for (n, k) in DSV3_NK for m in DSV3_M]

    def run_one(m, n, k, rot):
        pool = weights[(n, k)]
        wq, ws = pool[rot % len(pool)] if m <= 128 else pool[0]
        xq, xs = acts[(m, k)]
        return flag_gems.w8a8_block_fp8_matmul(xq, wq, xs, ws, [128, 128])

    if args.counter_pass:
        src = torch.randint(0, 255, (256 << 20,), device=dev, dtype=torch.uint8)
        dst = torch.empty_like(src)
        shapes = [(m, n, k) for (n, k) in DSV3_NK for m in DETAIL_M]
        for (m, n, k) in shapes:  # first launches (workspace zero fill etc.) happen before the counted ones
            run_one(m, n, k, 0)
        mark = torch.zeros(64, device=dev)
        torch.cuda.synchronize()
        dst.copy_(src)
        for (m, n, k) in shapes:
            mark.add_(1.0)  # an elementwise kernel between two calls: delimits the kernels of a call in the counter files
            run_one(m, n, k, 1)
        mark.add_(1.0)
        flag_gems.act_quant_triton(torch.randn(4096, 7168, device=dev, generator=gen).bfloat16(), 128)
        torch.cuda.synchronize()
        print("counter pass done: copy 268435456 B, then (M,N,K) =", shapes, "each after one elementwise marker kernel, "
              "then a marker and act_quant [4096,7168]", flush=True)
        return

    # The sweep is replayed from HIP graphs (the reference's benchmark harness has the same mode):
    # decode-sized GEMMs take a few microseconds on the GPU, less than a Python call takes on the host.
    # Each of the NG step graphs uses different copies of the small-M weights.
    NG = 4
    side = torch.cuda.Stream()
    step_graphs = []
    with torch.cuda.stream(side):
        for (m, n, k) in calls:  # warm every kernel variant and workspace on the capture stream
            run_one(m, n, k, 0)
        torch.cuda.synchronize()
        for gi in range(NG):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                for ci, (m, n, k) in enumerate(calls):
                    run_one(m, n, k, gi * 7 + ci)
            step_graphs.append(g)
    torch.cuda.synchronize()

    def run_step(i):
        for r in range(SWEEPS_PER_STEP):
            step_graphs[(i * SWEEPS_PER_STEP + r) % NG].replay()

    for i in range(args.warmup):
        run_step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        run_step(i)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    total_flops = SWEEPS_PER_STEP * sum(gemm_flops(*c) for c in calls)
    value = total_flops / (ms_per_step * 1e-3) / 1e12

    # ---- per-shape kernel time: HIP events (on the replay stream) around a graph of LAUNCHES back-to-back launches,
    # REPEATS replays, the first dropped, median of the rest
    def time_graph(fn_of_launch, launches=LAUNCHES, repeats=REPEATS):
        with torch.cuda.stream(side):
            fn_of_launch(0)
            fn_of_launch(1)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                for r in range(launches):
                    fn_of_launch(r)
        torch.cuda.synchronize()
        times = []
        for _ in range(repeats):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            g.replay()
            end.record()
            end.synchronize()
            times.append(start.elapsed_time(end) * 1e3 / launches)
        del g
        rest = sorted(times[1:])
        return rest[len(rest) // 2]

    # the floor for the weight-streaming kernels: a kernel that only reads a buffer of the weight's size once, launched
    # and rotated through the same pool exactly like the GEMM (fg_stream_read_probe)
    from flaggems_amd import _lib as fg_lib

    probe = fg_lib.load().fg_stream_read_probe
    sink = torch.zeros(4, dtype=torch.int32, device=dev)

    def read_probe(n, k, rot):
        pool = weights[(n, k)]
        wq = pool[rot % len(pool)][0]
        rc = probe(wq.data_ptr(), wq.numel(), sink.data_ptr(), torch.cuda.current_stream(dev).cuda_stream)
        assert rc == 0

    read_floor = {}
    for (n, k) in DSV3_NK:
        read_floor[(n, k)] = time_graph(lambda r: read_probe(n, k, r))

    detail = []
    for (n, k) in DSV3_NK:
        for m in DETAIL_M:
            us = time_graph(lambda r: run_one(m, n, k, r))
            tf = gemm_flops(m, n, k) / (us * 1e-6) / 1e12
            gbs = gemm_bytes(m, n, k) / (us * 1e-6) / 1e9
            row = {"M": m, "N": n, "K": k, "us": round(us, 2), "tflops": round(tf, 1), "gbps": round(gbs, 1),
                   "frac_mfma": round(tf / PEAK_FP8_TFLOPS, 4), "frac_hbm": round(gbs / PEAK_HBM_GBPS, 4)}
            if m <= 64:
                row["weight_read_floor_us"] = round(read_floor[(n, k)], 2)
                row["read_floor_over_us"] = round(read_floor[(n, k)] / us, 4)
            detail.append(row)

    # what the matrix pipes take of the kernel's own multiply phase when nothing else happens (fg_mfma_issue_probe:
    # operands in registers, no LDS, no memory), on the bytes of a quantized weight of the sweep: the part holds a
    # lower clock under matrix load than the one the published peak assumes
    mfma_probe = fg_lib.load().fg_mfma_issue_probe
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    probe_ops = weights[DSV3_NK[0]][0][0]

    def mfma_ceiling(with_fmas):
        iters = 1500  # ~2.5 ms: long enough for the clock to settle
        stream = torch.cuda.current_stream(dev).cuda_stream
        best = float("inf")
        for rep in range(4):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            assert mfma_probe(probe_ops.data_ptr(), iters, with_fmas, None, stream) == 0
            end.record()
            end.synchronize()
            if rep > 0:
                best = min(best, start.elapsed_time(end) * 1e-3)
        return iters * 32 * 65536.0 * 8 * cus / best / 1e12

    ceiling_block = mfma_ceiling(1)
    ceiling_plain = mfma_ceiling(0)

    big = [d for d in detail if d["M"] == 4096]
    big_flops = sum(gemm_flops(d["M"], d["N"], d["K"]) for d in big)
    big_time = sum(d["us"] for d in big) * 1e-6
    achieved = big_flops / big_time / 1e12
    traffic = sum(f + w for (f, w) in TRAFFIC_M4096_KIB.values()) * 1024.0 / len(TRAFFIC_M4096_KIB)
    roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_FP8_TFLOPS, 4), "traffic": round(traffic),
                "traffic_unit": "bytes per launch, mean of the six launches",
                "traffic_source": "profiles/fp8_gemm_dsv3_hbm_counters.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of "
                                  "`bench.py --counter-pass`, scaled by a 256 MiB copy in the same run; not re-measured in this run)",
                "flops_per_launch": big_flops / len(big), "algorithmic_bytes_per_launch":
                    sum(gemm_bytes(d["M"], d["N"], d["K"]) for d in big) / len(big),
                "avg_launch_us": round(big_time * 1e6 / len(big), 2),
                "kernel": "fp8_gemm_pingpong_kernel (with the scale transposition that precedes it), the six M=4096 calls of the sweep",
                "mfma_issue_ceiling": {
                    "block_scaled_mix": round(ceiling_block, 1), "mfma_only": round(ceiling_plain, 1), "unit": "TFLOP/s",
                    "frac_of_block_scaled_mix": round(achieved / ceiling_block, 4),
                    "what": "fg_mfma_issue_probe measured in this run: the kernel's multiply phase alone (8 wavefronts per "
                            "compute unit, MFMA 16x16x128 e4m3 on a quantized weight's bytes held in registers, with / "
                            "without the four scale FMAs per MFMA; no LDS, no memory, no barriers)"}}
    small = [d for d in detail if d["M"] <= 16]
    small_bytes = sum(gemm_bytes(d["M"], d["N"], d["K"]) for d in small)
    small_time = sum(d["us"] for d in small) * 1e-6
    roofline_small = {"bound": "hbm", "achieved": round(small_bytes / small_time / 1e9, 1), "peak": PEAK_HBM_GBPS,
                      "unit": "GB/s", "frac": round(small_bytes / small_time / 1e9 / PEAK_HBM_GBPS, 4),
                      "kernel": "the eighteen M in {1, 8, 16} launches of the six DSv3 (N,K), weights rotated through 512 MB",
                      "weight_read_floor_gbps": round(sum(n * k for (n, k) in DSV3_NK) / sum(read_floor.values()) / 1e3, 1),
                      "weight_read_floor_us": {f"{n}x{k}": round(v, 2) for (n, k), v in read_floor.items()},
                      "time_of_read_floor_over_time": round(3 * sum(read_floor.values()) / (small_time * 1e6), 4)}

    # ---- quantizer (HBM bound): act_quant on bf16 [4096, 7168]
    xq_in = torch.randn(4096, 7168, device=dev, generator=gen).bfloat16()
    for _ in range(3):
        flag_gems.act_quant_triton(xq_in, 128)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(50):
        flag_gems.act_quant_triton(xq_in, 128)
    end.record()
    end.synchronize()
    q_us = start.elapsed_time(end) * 1e3 / 50
    q_gbs = 3.03125 * 4096 * 7168 / (q_us * 1e-6) / 1e9
    quant = {"shape": [4096, 7168], "us": round(q_us, 2), "gbps": round(q_gbs, 1), "frac_hbm": round(q_gbs / PEAK_HBM_GBPS, 4)}

    # ---- 128 x 128 weight quantizer (HBM bound): bf16 [28672, 4096] -> e4m3fn + one scale per block
    w_in = (0.02 * torch.randn(28672, 4096, device=dev, generator=gen)).bfloat16()
    for _ in range(3):
        flag_gems.per_block_cast_to_fp8(w_in, use_ue8m0=False)
    torch.cuda.synchronize()
    start.record()
    for _ in range(20):
        flag_gems.per_block_cast_to_fp8(w_in, use_ue8m0=False)
    end.record()
    end.synchronize()
    wq_us = start.elapsed_time(end) * 1e3 / 20
    wq_gbs = (3.0 + 4.0 / 16384) * 28672 * 4096 / (wq_us * 1e-6) / 1e9
    weight_quant = {"shape": [28672, 4096], "us": round(wq_us, 2), "gbps": round(wq_gbs, 1),
                    "frac_hbm": round(wq_gbs / PEAK_HBM_GBPS, 4)}
    del w_in

    # ---- activation fused into the quantizer (HBM bound): bf16 [8192, 2 x 14336] gate|up -> e4m3fn [8192, 14336],
    # next to the two separate kernels it replaces
    gu = torch.randn(8192, 2 * 14336, device=dev, generator=gen).bfloat16()

    def time_calls(fn, reps=20):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        start.record()
        for _ in range(reps):
            fn()
        end.record()
        end.synchronize()
        return start.elapsed_time(end) * 1e3 / reps

    fused_us = time_calls(lambda: flag_gems.silu_and_mul_per_token_group_quant_fp8(gu, 128))
    apart_us = time_calls(lambda: flag_gems.per_token_group_quant_fp8(flag_gems.silu_and_mul_packed(gu), 128))
    fused_gbs = (5.0 + 4.0 / 128) * 8192 * 14336 / (fused_us * 1e-6) / 1e9
    fused = {"shape": [8192, 28672], "us": round(fused_us, 2), "gbps": round(fused_gbs, 1),
             "frac_hbm": round(fused_gbs / PEAK_HBM_GBPS, 4), "two_kernels_us": round(apart_us, 2)}
    del gu

    # ---- RMSNorm fused into the quantizer (HBM bound): bf16 [4096, 7168] -> e4m3fn codes + 1x128 scales, with and
    # without the residual add; algorithmic bytes per element: 2 read + 1 written (+ 4 / 128 of scales), and another
    # 2 read + 2 written for the residual
    hx = torch.randn(4096, 7168, device=dev, generator=gen).bfloat16()
    hr = torch.randn(4096, 7168, device=dev, generator=gen).bfloat16()
    hw = torch.ones(7168, device=dev, dtype=torch.bfloat16)
    norm_us = time_calls(lambda: flag_gems.rms_norm_per_token_group_quant_fp8(hx, hw, 128, eps=1e-6), 50)
    norm_apart_us = time_calls(lambda: flag_gems.per_token_group_quant_fp8(flag_gems.rms_norm(hx, (7168,), hw, 1e-6), 128), 50)
    hr.zero_()  # the residual accumulates x at every call: keep it finite
    add_us = time_calls(lambda: flag_gems.rms_norm_per_token_group_quant_fp8(hx, hw, 128, eps=1e-6, residual=hr.zero_()), 50)
    zero_us = time_calls(lambda: hr.zero_(), 50)
    norm_gbs = (3.0 + 4.0 / 128) * 4096 * 7168 / (norm_us * 1e-6) / 1e9
    add_gbs = (7.0 + 4.0 / 128) * 4096 * 7168 / ((add_us - zero_us) * 1e-6) / 1e9
    norm_quant = {"shape": [4096, 7168], "us": round(norm_us, 2), "gbps": round(norm_gbs, 1),
                  "frac_hbm": round(norm_gbs / PEAK_HBM_GBPS, 4), "two_kernels_us": round(norm_apart_us, 2),
                  "with_residual_us": round(add_us - zero_us, 2), "with_residual_gbps": round(add_gbs, 1),
                  "with_residual_frac_hbm": round(add_gbs / PEAK_HBM_GBPS, 4)}
    del hx, hr, hw

    # ---- the other configurations of the path, each shape timed alone: HIP events around the replay of a graph
    # of `reps` launches (as above: decode-sized launches are shorter than a Python call)
    def time_eager(fn, reps):
        return time_graph(lambda r: fn(), launches=max(reps, 20))

    # inverse RoPE fused into the group quantizer, the largest shape of the reference's benchmark
    # (benchmark/core_shapes.yaml "fused_inv_rope_fp8_quant": 4096 tokens, 128 heads of 512 in 8 groups, bf16)
    rope_tokens, rope_heads = 4096, 128
    r_o = torch.randn(rope_tokens, rope_heads, 512, device=dev, generator=gen).bfloat16()
    r_pos = torch.randint(0, 8192, (rope_tokens,), device=dev, generator=gen)
    r_freq = torch.outer(torch.arange(8192, dtype=torch.float32), 1.0 / (10000.0 ** (torch.arange(0, 32, dtype=torch.float32) / 32)))
    r_cache = torch.cat((r_freq.cos(), r_freq.sin()), dim=-1).to(dev)
    rope_bytes = rope_tokens * rope_heads * 512 * 3 + rope_tokens * rope_heads * 4 * 4
    rope_us = time_eager(lambda: flag_gems.fused_inv_rope_fp8_quant(r_o, r_pos, r_cache, 8, rope_heads // 8), 10)
    rope_packed_us = time_eager(lambda: flag_gems.fused_inv_rope_fp8_quant(r_o, r_pos, r_cache, 8, rope_heads // 8,
                                                                             tma_aligned_scales=True), 10)
    inv_rope = {"shape": [rope_tokens, rope_heads, 512], "groups": 8, "us": round(rope_us, 2),
                "gbps": round(rope_bytes / rope_us / 1e3, 1), "frac_hbm": round(rope_bytes / rope_us / 1e3 / PEAK_HBM_GBPS, 4),
                "packed_ue8m0_us": round(rope_packed_us, 2)}
    del r_o, r_pos, r_cache

    # routing in front of the expert layer: softmax + top-2 of 8 experts (Mixtral), group-limited top-8 of 256 experts in 8
    # groups (DeepSeek-V3), 4096 tokens each; latency-bound launches, reported in microseconds only
    rt_tokens = 4096
    rt_g8 = torch.randn(rt_tokens, 8, device=dev, generator=gen)
    rt_w = torch.empty(rt_tokens, 2, device=dev)
    rt_i = torch.empty(rt_tokens, 2, device=dev, dtype=torch.int32)
    rt_s = torch.empty(rt_tokens, 2, device=dev, dtype=torch.int32)
    rt_softmax_us = time_eager(lambda: flag_gems.topk_softmax(rt_w, rt_i, rt_s, rt_g8, True), 20)
    rt_g256 = torch.randn(rt_tokens, 256, device=dev, generator=gen).bfloat16()
    rt_bias = torch.randn(256, device=dev, generator=gen).bfloat16()
    rt_grouped_us = time_eager(lambda: flag_gems.grouped_topk(rt_g256, 8, 4, 8, True, 2.5, rt_bias, 1), 20)
    routing = {"tokens": rt_tokens, "topk_softmax_8_experts_top2_us": round(rt_softmax_us, 2),
               "grouped_topk_256_experts_8_groups_top8_us": round(rt_grouped_us, 2)}
    del rt_g8, rt_g256

    # the M = 4096 GEMMs of the sweep once more with power-of-two scales (ue8m0 quantization: act_quant scale_fmt
    # "ue8m0", per_block_cast_to_fp8 use_ue8m0), through the entry point that hands the scales to the matrix
    # instruction; the same call without that promise beside it
    pow2 = []
    for (n, k) in DSV3_NK:
        x = torch.randn(4096, k, device=dev, generator=gen).bfloat16()
        xq2, xs2 = flag_gems.act_quant_triton(x, 128, "ue8m0")
        w = (0.02 * torch.randn(n, k, device=dev, generator=gen)).bfloat16()
        wq2, ws2 = flag_gems.per_block_cast_to_fp8(w, use_ue8m0=True)
        del x, w
        us_plain = time_eager(lambda: flag_gems.w8a8_block_fp8_matmul(xq2, wq2, xs2, ws2, [128, 128]), 20)
        us_pow2 = time_eager(lambda: flag_gems.w8a8_block_fp8_matmul(xq2, wq2, xs2, ws2, [128, 128], scales_are_powers_of_two=True), 20)
        pow2.append({"M": 4096, "N": n, "K": k, "us": round(us_pow2, 2), "tflops": round(gemm_flops(4096, n, k) / us_pow2 / 1e6, 1),
                     "frac_mfma": round(gemm_flops(4096, n, k) / us_pow2 / 1e6 / PEAK_FP8_TFLOPS, 4),
                     "us_without_the_promise": round(us_plain, 2)})
        del xq2, xs2, wq2, ws2
    pow2_total = sum(r["us"] for r in pow2)
    pow2_summary = {"rows": pow2, "tflops": round(sum(gemm_flops(4096, n, k) for (n, k) in DSV3_NK) / pow2_total / 1e6, 1),
                    "frac_mfma": round(sum(gemm_flops(4096, n, k) for (n, k) in DSV3_NK) / pow2_total / 1e6 / PEAK_FP8_TFLOPS, 4),
                    "note": "not the headline configuration: scales restricted to powers of two"}

    # cutlass_scaled_mm semantics: per-token x per-channel scales, bf16 bias, N = K = 8192
    scaled = []
    nk = 8192
    b_src = torch.randn(nk, nk, device=dev, generator=gen)
    b_s = (b_src.abs().amax(dim=1) / 448.0).contiguous()
    b_q = (b_src / b_s[:, None]).to(torch.float8_e4m3fn)
    del b_src
    bias = torch.randn(nk, device=dev, generator=gen).bfloat16()
    for m in (1, 32, 256, 2048, 8192):
        a_src = torch.randn(m, nk, device=dev, generator=gen)
        a_s = (a_src.abs().amax(dim=1, keepdim=True) / 448.0).contiguous()
        a_q = (a_src / a_s).to(torch.float8_e4m3fn)
        c = torch.empty(m, nk, dtype=torch.bfloat16, device=dev)
        us = time_eager(lambda: flag_gems.cutlass_scaled_mm(c, a_q, b_q.t(), a_s, b_s.view(1, nk), bias), 10 if m >= 2048 else 30)
        nbytes = m * nk + nk * nk + 4 * m + 4 * nk + 2 * m * nk + 2 * nk
        scaled.append({"M": m, "N": nk, "K": nk, "us": round(us, 2), "tflops": round(gemm_flops(m, nk, nk) / us / 1e6, 1),
                       "gbps": round(nbytes / us / 1e3, 1)})
    del b_q, a_q, c

    # the int8 branch of cutlass_scaled_mm on the same shapes (the reference's int8 inputs: round(clamp(randn * 5)))
    scaled_i8 = []
    b_i8 = torch.round((torch.randn(nk, nk, device=dev, generator=gen) * 5).clamp(-128, 127)).to(torch.int8)
    b_si = torch.rand(nk, device=dev, generator=gen) * 0.02 + 0.001
    for m in (1, 32, 256, 2048, 8192):
        a_i8 = torch.round((torch.randn(m, nk, device=dev, generator=gen) * 5).clamp(-128, 127)).to(torch.int8)
        a_si = torch.rand(m, 1, device=dev, generator=gen) * 0.02 + 0.001
        c = torch.empty(m, nk, dtype=torch.bfloat16, device=dev)
        us = time_eager(lambda: flag_gems.cutlass_scaled_mm(c, a_i8, b_i8.t(), a_si, b_si.view(1, nk), bias), 10 if m >= 2048 else 30)
        nbytes = m * nk + nk * nk + 4 * m + 4 * nk + 2 * m * nk + 2 * nk
        scaled_i8.append({"M": m, "N": nk, "K": nk, "us": round(us, 2), "tops": round(gemm_flops(m, nk, nk) / us / 1e6, 1),
                          "gbps": round(nbytes / us / 1e3, 1)})
    del b_i8, a_i8, c

    # aten::_scaled_mm on operands that are not quantized (the generic kernel): per-row x per-column scales, N = K = 4096
    generic = []
    for dt, peak in ((torch.bfloat16, 2500.0), (torch.float16, 2500.0), (torch.float32, 157.3)):
        gb = torch.randn(4096, 4096, device=dev, generator=gen).to(dt).t()
        g_sb = torch.rand(1, 4096, device=dev, generator=gen) + 0.5
        for m in (1, 64, 4096):
            ga = torch.randn(m, 4096, device=dev, generator=gen).to(dt)
            g_sa = torch.rand(m, 1, device=dev, generator=gen) + 0.5
            us = time_eager(lambda: flag_gems.scaled_mm(ga, gb, g_sa, g_sb), 10)
            tf = gemm_flops(m, 4096, 4096) / us / 1e6
            g_bytes = (m * 4096 + 4096 * 4096 + m * 4096) * ga.element_size()
            generic.append({"dtype": str(dt)[6:], "M": m, "N": 4096, "K": 4096, "us": round(us, 2), "tflops": round(tf, 1),
                            "gbps": round(g_bytes / us / 1e3, 1), "frac_mfma": round(tf / peak, 4)})
        del ga, gb

    # fp8_einsum("bhr,hdr->bhd") at the first shape group of the reference's benchmark (h = 8, r = 4096, d = 1024)
    einsum = []
    eh, er, ed = 8, 4096, 1024
    ey = torch.randn(eh, ed, er, device=dev, generator=gen).to(torch.float8_e4m3fn)
    eys = torch.rand(eh, ed // 128, er // 128, device=dev, generator=gen) + 0.5
    for eb in (1, 128, 4096):
        ex = torch.randn(eb, eh, er, device=dev, generator=gen).to(torch.float8_e4m3fn)
        exs = torch.rand(eb, eh, er // 128, device=dev, generator=gen) + 0.5
        us = time_eager(lambda: flag_gems.fp8_einsum("bhr,hdr->bhd", ex, exs, ey, eys), 10)
        nbytes = eh * ed * er + eb * eh * er + 2 * eb * eh * ed + 4 * (eh * (ed // 128) * (er // 128) + eb * eh * (er // 128))
        tf = 2.0 * eb * eh * ed * er / us / 1e6
        einsum.append({"b": eb, "h": eh, "r": er, "d": ed, "us": round(us, 2), "tflops": round(tf, 1),
                       "gbps": round(nbytes / us / 1e3, 1), "frac_mfma": round(tf / PEAK_FP8_TFLOPS, 4),
                       "frac_hbm": round(nbytes / us / 1e3 / PEAK_HBM_GBPS, 4)})
    del ey, eys, ex, exs

    # Llama-3-8B linears: GEMM alone and act_quant + GEMM from bf16 activations; for M <= 128 every launch reads another
    # copy of the weights out of a pool of at least 512 MB, as in the sweep above
    llama = []
    for (n, k) in [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]:
        wq, ws = make_weight(n, k, gen, dev)
        copies = max(1, -(-CACHE_BYTES // (n * k)))
        pool = [wq] + [wq.clone() for _ in range(copies - 1)]
        for m in (1, 16, 128, 1024, 4096):
            x = torch.randn(m, k, device=dev, generator=gen).bfloat16()
            xq, xs = flag_gems.act_quant_triton(x, 128)
            use = pool if m <= 128 else pool[:1]
            launches = LAUNCHES if m <= 1024 else 20
            us_g = time_graph(lambda r: flag_gems.w8a8_block_fp8_matmul(xq, use[r % len(use)], xs, ws, [128, 128]), launches)

            def e2e(r):
                q, s2 = flag_gems.act_quant_triton(x, 128)
                return flag_gems.w8a8_block_fp8_matmul(q, use[r % len(use)], s2, ws, [128, 128])

            us_e = time_graph(e2e, launches)
            llama.append({"M": m, "N": n, "K": k, "gemm_us": round(us_g, 2), "quant_gemm_us": round(us_e, 2),
                          "tflops": round(gemm_flops(m, n, k) / us_g / 1e6, 1), "gbps": round(gemm_bytes(m, n, k) / us_g / 1e3, 1),
                          "weight_copies": len(use)})
        del wq, ws, pool

    # the row counts at which one kernel hands over to the next (16/17: decode kernels / two parts of up to 16 rows; 32/33: to
    # the staged-activation kernel; 64/65: to two halves of it, or the K-split tile kernel; 128/129: tile kernel), weights rotated
    handover = []
    for (n, k) in [(2112, 7168), (4096, 4096), (7168, 16384)]:
        wq, ws = make_weight(n, k, gen, dev)
        copies = max(1, -(-CACHE_BYTES // (n * k)))
        pool = [wq] + [wq.clone() for _ in range(copies - 1)]
        row = {"N": n, "K": k, "us_by_rows": {}}
        for m in (16, 17, 32, 33, 64, 65, 128, 129):
            xq = torch.randn(m, k, device=dev, generator=gen).to(torch.float8_e4m3fn)
            xs = torch.rand(m, k // 128, device=dev, generator=gen) + 0.5
            us = time_graph(lambda r: flag_gems.w8a8_block_fp8_matmul(xq, pool[r % len(pool)], xs, ws, [128, 128]))
            row["us_by_rows"][str(m)] = round(us, 2)
        handover.append(row)
        del wq, ws, pool

    # Mixtral-8x7B expert layers: grouped block-fp8 GEMM over rows sorted by expert
    moe = []
    experts = 8
    moe_w = {}
    for (n, k) in [(28672, 4096), (4096, 14336)]:
        parts = [make_weight(n, k, gen, dev) for _ in range(experts)]
        wq = torch.stack([q for (q, _) in parts])
        ws = torch.stack([s_ for (_, s_) in parts])
        del parts
        moe_w[(n, k)] = (wq, ws)
        for tokens in (64, 1024, 4096):
            rows = 2 * tokens
            ends = moe_row_ends(tokens, experts, 2, 0).to(dev)
            xq, xs = flag_gems.act_quant_triton(torch.randn(rows, k, device=dev, generator=gen).bfloat16(), 128)
            us = time_eager(lambda: flag_gems.grouped_w8a8_block_fp8_matmul(xq, wq, xs, ws, ends, [128, 128]), 10)
            nbytes = experts * (n * k + 4 * (n // 128) * (k // 128)) + rows * k + 4 * rows * (k // 128) + 2 * rows * n
            tf = gemm_flops(rows, n, k) / us / 1e6
            moe.append({"tokens": tokens, "rows": rows, "N": n, "K": k, "row_ends": ends.tolist(), "us": round(us, 2),
                        "tflops": round(tf, 1), "gbps": round(nbytes / us / 1e3, 1),
                        "frac_mfma": round(tf / PEAK_FP8_TFLOPS, 4), "frac_hbm": round(nbytes / us / 1e3 / PEAK_HBM_GBPS, 4)})
        del wq, ws

    # the whole expert layer: quantize -> grouped GEMM 1 (gather) -> SiLU-and-mul + quantize -> grouped GEMM 2 (scatter,
    # routing weight) -> sum over the two slots of a token (fused_experts_impl), bf16 [T, 4096] in and out, the same
    # Zipf(1.1) expert loads; flops = 2 * 2T * (28672 * 4096 + 4096 * 14336)
    moe_layer = []
    (w1q, w1s), (w2q, w2s) = moe_w[(28672, 4096)], moe_w[(4096, 14336)]
    for tokens in (64, 1024, 4096):
        ends = moe_row_ends(tokens, experts, 2, 0)
        counts = torch.diff(ends, prepend=torch.zeros(1, dtype=torch.int32))
        ids = torch.repeat_interleave(torch.arange(experts), counts.long())
        ids = ids[torch.randperm(ids.numel(), generator=torch.Generator().manual_seed(tokens))].view(tokens, 2).to(dev)
        tw = torch.rand(tokens, 2, device=dev, generator=gen) + 0.1
        tw = (tw / tw.sum(dim=1, keepdim=True)).bfloat16()
        hs = torch.randn(tokens, 4096, device=dev, generator=gen).bfloat16()
        us = time_eager(lambda: flag_gems.fused_experts_impl(hs, w1q, w2q, tw, ids, use_fp8_w8a8=True, w1_scale=w1s,
                                                             w2_scale=w2s, block_shape=[128, 128]), 10)
        fl = 2.0 * 2 * tokens * (28672 * 4096 + 4096 * 14336)
        gemm_rows = [r for r in moe if r["tokens"] == tokens]
        moe_layer.append({"tokens": tokens, "us": round(us, 2), "tflops": round(fl / us / 1e6, 1),
                          "frac_mfma": round(fl / us / 1e6 / PEAK_FP8_TFLOPS, 4),
                          "weight_gbps": round(experts * (28672 * 4096 + 4096 * 14336) / us / 1e3, 1),
                          "the_two_gemms_alone_us": round(sum(r["us"] for r in gemm_rows), 2)})
    del moe_w, w1q, w1s, w2q, w2s

    # ---- host time of an eager call (no graph): what a decode step pays per launch on the host, next to the kernel's
    # own time.  fp8_matmul = checks + allocation + launch; fp8_matmul_noop = checks + allocation (the reference's
    # probe of its binding overhead, cpp/lib/fp8_matmul.cpp:104-125); the bare C-ABI call through ctypes with all
    # arguments prepared = the launch alone.  Host time = wall time of enqueueing, the queue never full (a
    # synchronisation every 200 calls, outside the clock).
    eager = []
    lib = fg_lib.load()
    for (n, k) in [(2112, 7168), (7168, 16384)]:
        xq, xs = acts[(1, k)]
        wq, ws = weights[(n, k)][0]

        def host_us(fn, calls=2000, burst=200):
            for _ in range(50):
                fn()
            torch.cuda.synchronize()
            spent = 0.0
            for _ in range(calls // burst):
                t0 = time.perf_counter()
                for _ in range(burst):
                    fn()
                spent += time.perf_counter() - t0
                torch.cuda.synchronize()
            return spent / calls * 1e6

        c = torch.empty(1, n, dtype=torch.bfloat16, device=dev)
        need = lib.fg_block_fp8_gemm_workspace_bytes(1, n, k)
        wsp = torch.zeros(max(need, 16384), dtype=torch.uint8, device=dev)
        raw = (xq.data_ptr(), k, wq.data_ptr(), k, xs.data_ptr(), xs.stride(0), xs.stride(1), ws.data_ptr(), ws.stride(0),
               ws.stride(1), c.data_ptr(), n, 0, 1, n, k, 128, 128, wsp.data_ptr(), wsp.numel(),
               fg_lib.current_stream_ptr(dev))
        kernel_us = [d["us"] for d in detail if (d["M"], d["N"], d["K"]) == (1, n, k)][0]
        eager.append({"M": 1, "N": n, "K": k,
                      "fp8_matmul_host_us": round(host_us(lambda: flag_gems.fp8_matmul(xq, xs, wq, ws)), 2),
                      "w8a8_block_fp8_matmul_host_us": round(host_us(lambda: flag_gems.w8a8_block_fp8_matmul(xq, wq, xs, ws, [128, 128])), 2),
                      "fp8_matmul_noop_host_us": round(host_us(lambda: flag_gems.fp8_matmul_noop(xq, xs, wq, ws)), 2),
                      "bare_c_abi_call_host_us": round(host_us(lambda: lib.fg_block_fp8_gemm(*raw)), 2),
                      "kernel_us_in_a_graph": kernel_us})
        del c, wsp

    # ---- CPU baseline: the oracle on the host cores, bounded samples
    cpu = None
    cpu_configs = None
    if not args.no_cpu:
        from oracle import fp8_linear_oracle as O

        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        torch.set_num_threads(cores)
        sample_m = 4096
        cpu_flops, cpu_time, passes = 0.0, 0.0, 0
        cpu_in = []
        for (n, k) in DSV3_NK:
            xq, xs = acts[(4096, k)]
            wq, ws = weights[(n, k)][0]
            cpu_in.append((n, k, xq[:sample_m].cpu(), xs[:sample_m].cpu(), wq.cpu(), ws.cpu()))
        while cpu_time < 10.0 and passes < 8:  # whole passes over the six GEMMs
            for (n, k, a, a_s, b, b_s) in cpu_in:
                t0 = time.perf_counter()
                O.block_fp8_matmul_tiled_ref(a, b, a_s, b_s, [128, 128], torch.bfloat16)
                cpu_time += time.perf_counter() - t0
                cpu_flops += gemm_flops(sample_m, n, k)
            passes += 1
        cpu = {"value": round(cpu_flops / cpu_time / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
               "sample": f"oracle block_fp8_matmul_tiled_ref (per-K-tile fp32 matmul, torch CPU) on the M={sample_m} "
                         f"GEMMs of the six DSv3 (N,K) shapes, {passes} passes, {cpu_time:.1f} s"}

        # the other configurations on the host, each timed once after one warm-up call (decode-sized M only: larger
        # ones take seconds per call on a CPU and say nothing new)
        def cpu_time_of(fn):
            fn()
            t0 = time.perf_counter()
            fn()
            return time.perf_counter() - t0

        cpu_configs = []
        x1, w1 = O.make_config1(0)
        t = cpu_time_of(lambda: O.run_config1(0))
        cpu_configs.append({"config": "1: act_quant + 128x128 weight quantizer + block-fp8 GEMM, M=64 N=512 K=1024, end to end",
                            "ms": round(t * 1e3, 3), "tflops": round(gemm_flops(64, 512, 1024) / t / 1e12, 5)})
        del x1, w1
        for (n, k, a, a_s, b, b_s) in cpu_in:
            m = 64
            t = cpu_time_of(lambda: O.block_fp8_matmul_tiled_ref(a[:m], b, a_s[:m], b_s, [128, 128], torch.bfloat16))
            cpu_configs.append({"config": f"3: DSv3 block-fp8 GEMM M={m} N={n} K={k}", "ms": round(t * 1e3, 3),
                                "tflops": round(gemm_flops(m, n, k) / t / 1e12, 5)})
        del cpu_in
        gcpu = torch.Generator().manual_seed(0)
        for (n, k) in [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]:
            m = 128
            xq_c, xs_c = O.act_quant_ref(torch.randn(m, k, generator=gcpu).bfloat16(), 128)
            wq_c, ws_c = O.per_block_cast_to_fp8_ref((0.02 * torch.randn(n, k, generator=gcpu)).bfloat16())
            t = cpu_time_of(lambda: O.block_fp8_matmul_tiled_ref(xq_c, wq_c, xs_c, ws_c, [128, 128], torch.bfloat16))
            cpu_configs.append({"config": f"2: Llama-3-8B linear M={m} N={n} K={k}", "ms": round(t * 1e3, 3),
                                "tflops": round(gemm_flops(m, n, k) / t / 1e12, 5)})
        m, nk_c = 32, 8192
        a_c = torch.randn(m, nk_c, generator=gcpu).clamp(-448, 448).to(torch.float8_e4m3fn)
        b_c = torch.randn(nk_c, nk_c, generator=gcpu).clamp(-448, 448).to(torch.float8_e4m3fn).t()
        sa_c, sb_c = torch.rand(m, 1, generator=gcpu), torch.rand(1, nk_c, generator=gcpu)
        bias_c = torch.randn(nk_c, generator=gcpu).bfloat16()
        t = cpu_time_of(lambda: O.scaled_mm_ref(a_c, b_c, sa_c, sb_c, torch.bfloat16, bias_c))
        cpu_configs.append({"config": f"4: cutlass_scaled_mm M={m} N={nk_c} K={nk_c} with bias", "ms": round(t * 1e3, 3),
                            "tflops": round(gemm_flops(m, nk_c, nk_c) / t / 1e12, 5)})

    out = {
        "metric": "block_fp8_gemm_tflops",
        "value": round(value, 1),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn x fp8_e4m3fn -> f32 accumulate -> bf16",
        "data": "synthetic",
        "config": {"workload": "DeepSeek-V3 block-fp8 GEMM sweep: M in {1,8,64,512,2048,4096} x 6 (N,K); "
                               "1x128 activation scales, 128x128 weight scales, bf16 out; one step = 16 passes over all 36 GEMMs, each pass one HIP graph replay "
                               "(weights of the M <= 64 calls rotated through 512 MB)",
                   "sweeps_per_step": SWEEPS_PER_STEP,
                   "pct_fp8_mfma_peak_at_M4096": round(100 * achieved / PEAK_FP8_TFLOPS, 2),
                   "pct_hbm_at_M_le_16": round(100 * roofline_small["frac"], 2)},
        "roofline": roofline,
        "roofline_small_m": roofline_small,
        "quantizer": quant,
        "weight_quantizer_128x128": weight_quant,
        "silu_mul_quantizer": fused,
        "rms_norm_quantizer": norm_quant,
        "inv_rope_quantizer": inv_rope,
        "moe_routing": routing,
        "block_fp8_gemm_pow2_scales_m4096": pow2_summary,
        "cutlass_scaled_mm_n8192_k8192_bias": scaled,
        "cutlass_scaled_mm_int8_n8192_k8192_bias": scaled_i8,
        "scaled_mm_unquantized_operands": generic,
        "fp8_einsum_bhr_hdr": einsum,
        "llama3_8b_linears": llama,
        "rows_at_the_hand_over_points": handover,
        "mixtral_moe_grouped_gemm": moe,
        "mixtral_moe_layer": moe_layer,
        "eager_host_overhead": eager,
        "cpu_baseline": cpu,
        "cpu_baseline_other_configs": cpu_configs,
        "detail": detail,
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
