"""fg_block_fp8_gemm_noalloc (the entry point whose workspace is a device array built into the library) against
fg_block_fp8_gemm given a workspace of the caller's: same kernels, so the same bits; and against the CPU oracle to
the GEMM bar (|got - want| <= 1e-2 + 1e-2 |want| on the bf16 result).  Two calls in a row share the built-in
array, the second with a smaller problem; both shapes split K between blocks, so both use counters and partial sums."""
import pytest
import torch

from flaggems_amd import _lib
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _problem(M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (0.02 * torch.randn(N, K, generator=g)).bfloat16()
    xq, xs = O.act_quant_ref(x, 128)
    wq, ws = O.per_block_cast_to_fp8_ref(w)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    return [t.to(DEV) for t in (xq, wq, xs, ws)], want


def _call(fn, ops, M, N, K, *tail):
    a, b, a_s, b_s = ops
    c = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    rc = fn(a.data_ptr(), K, b.data_ptr(), K, a_s.data_ptr(), a_s.stride(0), a_s.stride(1),
            b_s.data_ptr(), b_s.stride(0), b_s.stride(1), c.data_ptr(), N, _lib.FG_BF16, M, N, K, 128, 128, *tail)
    return rc, c


def test_noalloc_entry_point_matches_the_workspace_entry_point():
    lib = _lib.load()
    stream = _lib.current_stream_ptr(torch.device(DEV))
    shapes = [(64, 2112, 7168), (8, 256, 8192), (300, 1300, 2048), (4096, 1024, 1024)]
    problems = [(_problem(M, N, K, 30 + i), (M, N, K)) for i, (M, N, K) in enumerate(shapes)]
    for round_ in range(2):  # the second pass finds the array as the first left it
        for (ops, want), (M, N, K) in problems:
            need = lib.fg_block_fp8_gemm_workspace_bytes(M, N, K)
            assert need <= _lib.FG_NOALLOC_SCRATCH_BYTES
            print(f"noalloc case M={M} N={N} K={K} workspace={need} pass={round_}", flush=True)
            rc, got = _call(lib.fg_block_fp8_gemm_noalloc, ops, M, N, K, stream)
            _lib.check(rc, "fg_block_fp8_gemm_noalloc")
            ws = torch.zeros(_lib.FG_NOALLOC_SCRATCH_BYTES, dtype=torch.uint8, device=DEV)
            rc, ref = _call(lib.fg_block_fp8_gemm, ops, M, N, K, ws.data_ptr(), ws.numel(), stream)
            _lib.check(rc, "fg_block_fp8_gemm")
            torch.cuda.synchronize()
            assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), (M, N, K)
            torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    assert lib.fg_block_fp8_gemm_workspace_bytes(64, 2112, 7168) > _lib.FG_WORKSPACE_COUNTER_BYTES
    assert lib.fg_block_fp8_gemm_workspace_bytes(8, 256, 8192) > _lib.FG_WORKSPACE_COUNTER_BYTES


def test_noalloc_entry_point_refuses_what_does_not_fit():
    lib = _lib.load()
    M, N, K = 128, 7168, 16384
    assert lib.fg_block_fp8_gemm_workspace_bytes(M, N, K) > _lib.FG_NOALLOC_SCRATCH_BYTES
    rc = lib.fg_block_fp8_gemm_noalloc(1, K, 1, K, 1, 1, 1, 1, 1, 1, 1, N, _lib.FG_BF16, M, N, K, 128, 128, None)
    assert rc == _lib.FG_ERR_WORKSPACE
    assert b"built-in buffer" in lib.fg_last_error_string()
    assert lib.fg_block_fp8_gemm_noalloc(None, 0, None, 0, None, 0, 0, None, 0, 0, None, 0, _lib.FG_BF16, 0, 8, 128, 128, 128, None) == 0


def test_noalloc_entry_point_under_graph_capture():
    """Launches recorded into a HIP graph (the callers the entry point is for), replayed several times with eager
    calls of the same entry point on the same stream in between: every replay and every eager call gives the bits of
    fg_block_fp8_gemm.  The shapes split K between blocks, so counters and partial sums of the built-in array are in
    use by every launch, recorded or not."""
    lib = _lib.load()
    shapes = [(64, 2112, 7168), (8, 256, 8192)]
    problems = [(_problem(M, N, K, 50 + i)[0], (M, N, K)) for i, (M, N, K) in enumerate(shapes)]
    side = torch.cuda.Stream()
    refs, outs = [], []
    with torch.cuda.stream(side):
        stream = _lib.current_stream_ptr(torch.device(DEV))
        for ops, (M, N, K) in problems:
            ws = torch.zeros(_lib.FG_NOALLOC_SCRATCH_BYTES, dtype=torch.uint8, device=DEV)
            rc, ref = _call(lib.fg_block_fp8_gemm, ops, M, N, K, ws.data_ptr(), ws.numel(), stream)
            _lib.check(rc, "fg_block_fp8_gemm")
            refs.append(ref)
            outs.append(torch.empty(M, N, dtype=torch.bfloat16, device=DEV))
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            stream = _lib.current_stream_ptr(torch.device(DEV))
            for (ops, (M, N, K)), c in zip(problems, outs):
                a, b, a_s, b_s = ops
                rc = lib.fg_block_fp8_gemm_noalloc(a.data_ptr(), K, b.data_ptr(), K, a_s.data_ptr(), a_s.stride(0), a_s.stride(1),
                                                   b_s.data_ptr(), b_s.stride(0), b_s.stride(1), c.data_ptr(), N, _lib.FG_BF16,
                                                   M, N, K, 128, 128, stream)
                _lib.check(rc, "fg_block_fp8_gemm_noalloc under capture")
        for replay in range(4):
            for c in outs:
                c.fill_(float("nan"))
            print(f"noalloc graph replay {replay}", flush=True)
            graph.replay()
            torch.cuda.synchronize()
            for c, ref in zip(outs, refs):
                assert torch.equal(c.view(torch.int16), ref.view(torch.int16)), f"replay {replay}"
            # eager work of the program's own between the replays, through the same built-in array
            stream = _lib.current_stream_ptr(torch.device(DEV))
            for (ops, (M, N, K)), ref in zip(problems, refs):
                rc, got = _call(lib.fg_block_fp8_gemm_noalloc, ops, M, N, K, stream)
                _lib.check(rc, "fg_block_fp8_gemm_noalloc")
                torch.cuda.synchronize()
                assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), f"eager call after replay {replay}"
