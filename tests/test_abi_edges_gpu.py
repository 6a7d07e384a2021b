"""GPU checks of the C ABI's corners: the act_quant stand-in called raw, power-of-two scales given as
float8_e8m0fnu, empty K, the host-only probe, and the workspace under HIP-graph capture."""
import pytest
import torch

import flag_gems
from flaggems_amd import _lib
from oracle import fp8_linear_oracle as O
from tests._util import assert_codes_equal, assert_scales_equal

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn


@pytest.mark.parametrize("round_scale", [0, 1])
@pytest.mark.parametrize("rows,cols", [(1, 128), (64, 1024), (300, 7168), (4096, 512)])
def test_fg_act_quant_bf16_through_ctypes(rows, cols, round_scale):
    """fg_act_quant_bf16 is the C-ABI counterpart of the reference's C++ wrapper (cpp/lib/act_quant.cpp:26-129,
    bound at cpp/csrc/cstub.cpp:81-85): bf16 in, e4m3fn codes and fp32 scales out, power-of-two scales when
    round_scale is set.  Bit-exact against the restated torch_act_quant (tests/test_act_quant.py:48-98)."""
    g = torch.Generator().manual_seed(rows + cols)
    x = (torch.randn(rows, cols, generator=g) * torch.logspace(-3, 2, rows).unsqueeze(1)).bfloat16()
    x[0, :3] = torch.tensor([0.0, -0.0, 448.0]).bfloat16()
    want_q, want_s = O.act_quant_ref(x, 128, "ue8m0" if round_scale else None)
    xd = x.to(DEV)
    q = torch.empty(rows, cols, dtype=FP8, device=DEV)
    s = torch.empty(rows, cols // 128, dtype=torch.float32, device=DEV)
    rc = _lib.load().fg_act_quant_bf16(xd.data_ptr(), q.data_ptr(), s.data_ptr(), rows, cols, 128, round_scale,
                                       _lib.current_stream_ptr(torch.device(DEV)))
    _lib.check(rc, "fg_act_quant_bf16")
    torch.cuda.synchronize()
    assert_codes_equal(q, want_q, "fg_act_quant_bf16 codes")
    assert_scales_equal(s, want_s, "fg_act_quant_bf16 scales")
    # and it is the kernel behind the Python entry point
    pq, ps = flag_gems.act_quant_triton(xd, 128, "ue8m0" if round_scale else None)
    assert torch.equal(pq.view(torch.uint8), q.view(torch.uint8)) and torch.equal(ps, s)


def test_fg_act_quant_bf16_rejects_bad_arguments():
    lib = _lib.load()
    x = torch.zeros(4, 256, dtype=torch.bfloat16, device=DEV)
    q = torch.empty(4, 256, dtype=FP8, device=DEV)
    s = torch.empty(4, 2, dtype=torch.float32, device=DEV)
    assert lib.fg_act_quant_bf16(x.data_ptr(), q.data_ptr(), s.data_ptr(), 4, 200, 128, 0, None) == _lib.FG_ERR_INVALID_ARG
    assert lib.fg_act_quant_bf16(None, q.data_ptr(), s.data_ptr(), 4, 256, 128, 0, None) == _lib.FG_ERR_INVALID_ARG
    assert lib.fg_act_quant_bf16(None, None, None, 0, 256, 128, 0, None) == 0


def test_fp8_matmul_takes_e8m0_scales():
    """scale_dtype=float8_e8m0fnu: the scales are widened to fp32 before the launch (reference
    src/flag_gems/ops/fp8_matmul.py:165-167), so the result equals the fp32-scale call bit for bit."""
    M, N, K = 48, 640, 1024
    g = torch.Generator().manual_seed(4)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (0.02 * torch.randn(N, K, generator=g)).bfloat16()
    xq, xs = O.act_quant_ref(x, 128, "ue8m0")
    wq, ws = O.per_block_cast_to_fp8_ref(w, use_ue8m0=True)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    a, b = xq.to(DEV), wq.to(DEV)
    xs8, ws8 = xs.to(DEV).to(torch.float8_e8m0fnu), ws.to(DEV).to(torch.float8_e8m0fnu)
    assert torch.equal(xs8.to(torch.float32).cpu(), xs) and torch.equal(ws8.to(torch.float32).cpu(), ws)
    got8 = flag_gems.fp8_matmul(a, xs8, b, ws8, scale_dtype=torch.float8_e8m0fnu)
    got32 = flag_gems.fp8_matmul(a, xs.to(DEV), b, ws.to(DEV))
    assert got8.dtype == torch.bfloat16 and got8.shape == (M, N)
    assert torch.equal(got8.view(torch.int16), got32.view(torch.int16))
    torch.testing.assert_close(got8.cpu().float(), want, rtol=1e-2, atol=1e-2)


def test_fp8_matmul_noop_checks_and_allocates_only():
    a = torch.zeros(2, 3, 256, dtype=FP8, device=DEV)
    b = torch.zeros(384, 256, dtype=FP8, device=DEV)
    a_s = torch.ones(2, 3, 2, device=DEV)
    b_s = torch.ones(3, 2, device=DEV)
    out = flag_gems.fp8_matmul_noop(a, a_s, b, b_s)
    assert out.shape == (2, 3, 384) and out.dtype == torch.bfloat16 and out.device.type == "cuda"
    with pytest.raises(AssertionError, match="same K"):
        flag_gems.fp8_matmul_noop(a, a_s, b[:, :128].contiguous(), b_s)
    with pytest.raises(AssertionError, match="contiguous"):
        flag_gems.fp8_matmul_noop(a, a_s, b.t(), b_s)


@pytest.mark.parametrize("M", [5, 100, 300])
def test_empty_k_gives_zeros_or_the_bias(M):
    """K = 0: an empty sum.  The block-scaled GEMM writes zeros, the row/column-scaled one the bias, whatever kernel
    the row count would otherwise select."""
    N = 512
    dev = torch.device(DEV)
    lib = _lib.load()
    c = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
    one = torch.ones(max(M, N), device=DEV)
    rc = lib.fg_block_fp8_gemm(None, 0, None, 0, None, 0, 1, None, 0, 1, c.data_ptr(), N, _lib.FG_BF16,
                               M, N, 0, 128, 128, None, 0, _lib.current_stream_ptr(dev))
    _lib.check(rc, "fg_block_fp8_gemm")
    torch.cuda.synchronize()
    assert (c == 0).all()
    bias = torch.randn(N, device=DEV).bfloat16()
    c.fill_(7.0)
    rc = lib.fg_scaled_fp8_gemm(None, 0, None, 0, one.data_ptr(), 1, one.data_ptr(), 1, bias.data_ptr(), _lib.FG_BF16,
                                c.data_ptr(), N, _lib.FG_BF16, M, N, 0, None, 0, _lib.current_stream_ptr(dev))
    _lib.check(rc, "fg_scaled_fp8_gemm")
    torch.cuda.synchronize()
    assert torch.equal(c, bias.unsqueeze(0).expand(M, N))


def _quantized(M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (0.02 * torch.randn(N, K, generator=g)).bfloat16()
    xq, xs = O.act_quant_ref(x, 128)
    wq, ws = O.per_block_cast_to_fp8_ref(w)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    return [t.to(DEV) for t in (xq, wq, xs, ws)], want


def test_workspace_outlives_the_graphs_that_captured_it():
    """A launch recorded into a HIP graph keeps the workspace address it was given.  A later call that needs a larger
    workspace must not release that memory: the first graph is replayed afterwards, with other allocations made in
    between, and must still give the oracle's result.  Covers both orders: workspace made before the capture (on the
    capture stream) and workspace made inside the capture."""
    small, want_small = _quantized(8, 256, 8192, 1)      # decode kernel with K split over blocks: uses the workspace
    big, want_big = _quantized(700, 1300, 8192, 2)       # persistent kernel sharing tiles along K: a much larger one
    lib = _lib.load()
    assert lib.fg_block_fp8_gemm_workspace_bytes(8, 256, 8192) > 0
    assert lib.fg_block_fp8_gemm_workspace_bytes(700, 1300, 8192) > 4 * lib.fg_block_fp8_gemm_workspace_bytes(8, 256, 8192)
    stream = torch.cuda.Stream()
    for warm_on_capture_stream in (True, False):
        _lib._workspaces.clear()
        if warm_on_capture_stream:
            with torch.cuda.stream(stream):
                flag_gems.w8a8_block_fp8_matmul(*small, [128, 128])
            stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            out_small = flag_gems.w8a8_block_fp8_matmul(*small, [128, 128])
        graph.replay()
        torch.cuda.synchronize()
        torch.testing.assert_close(out_small.cpu().float(), want_small, rtol=1e-2, atol=1e-2)
        first = out_small.clone()
        # eager calls on the same stream that outgrow the workspace, and allocations that would reuse freed memory
        with torch.cuda.stream(stream):
            out_big = flag_gems.w8a8_block_fp8_matmul(*big, [128, 128])
            junk = [torch.full((1 << 20,), 1e30, device=DEV) for _ in range(64)]
        stream.synchronize()
        torch.testing.assert_close(out_big.cpu().float(), want_big, rtol=1e-2, atol=1e-2)
        for _ in range(3):
            out_small.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out_small, first)
        with torch.cuda.stream(stream):
            again = flag_gems.w8a8_block_fp8_matmul(*big, [128, 128])
        stream.synchronize()
        assert torch.equal(again, out_big)
        del junk, graph


@pytest.mark.parametrize("M,N,K", [(1, 2112, 7168), (16, 24576, 1536), (8, 7168, 2304), (16, 4096, 4096)])
def test_decode_kernels_replayed_from_a_graph(M, N, K):
    """The decode kernels in their three forms (activations copied into LDS per wavefront, a wavefront per 16 rows of
    wide weights, activation fragments in registers) give, replayed from a HIP graph several times with eager work
    between the replays, the bits of the eager call."""
    args, want = _quantized(M, N, K, 5)
    eager = flag_gems.w8a8_block_fp8_matmul(*args, [128, 128])
    torch.testing.assert_close(eager.cpu().float(), want, rtol=1e-2, atol=1e-2)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        out = flag_gems.w8a8_block_fp8_matmul(*args, [128, 128])
    for _ in range(3):
        out.zero_()
        other = flag_gems.w8a8_block_fp8_matmul(args[0], args[1], args[2] * 2, args[3], [128, 128])  # eager work in between
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        assert not torch.equal(other, eager)


def test_measurement_probes_run_and_check_their_arguments():
    """fg_stream_read_probe and fg_mfma_issue_probe are what bench.py puts its figures next to: both must run on any
    input they accept and refuse what they cannot take."""
    lib = _lib.load()
    stream = _lib.current_stream_ptr(torch.device(DEV))
    buf = torch.randint(0, 255, (1 << 20,), dtype=torch.uint8, device=DEV)
    sink = torch.zeros(4, dtype=torch.int32, device=DEV)
    assert lib.fg_stream_read_probe(buf.data_ptr(), buf.numel(), sink.data_ptr(), stream) == 0
    assert lib.fg_stream_read_probe(buf.data_ptr(), 0, None, stream) == 0
    assert lib.fg_stream_read_probe(buf.data_ptr() + 8, 1024, None, stream) == _lib.FG_ERR_INVALID_ARG
    for with_fmas in (0, 1):
        assert lib.fg_mfma_issue_probe(buf.data_ptr(), 3, with_fmas, None, stream) == 0
        assert lib.fg_mfma_issue_probe(buf.data_ptr(), 1, with_fmas, sink.data_ptr(), stream) == 0
    assert lib.fg_mfma_issue_probe(None, 3, 1, None, stream) == _lib.FG_ERR_INVALID_ARG
    assert lib.fg_mfma_issue_probe(buf.data_ptr() + 8, 3, 1, None, stream) == _lib.FG_ERR_INVALID_ARG
    assert lib.fg_mfma_issue_probe(buf.data_ptr(), 0, 1, None, stream) == _lib.FG_ERR_INVALID_ARG
    torch.cuda.synchronize()
    assert int(sink.abs().sum()) == 0  # the sinks are written for no real input
