"""GPU parity of the block-scaled FP8 GEMM against the CPU oracle.

Tolerance: rtol 1e-2 / atol 1e-2 (the bar this build sets itself) against the fp32-dequantised matmul for bf16 output;
the reference's own tolerance (fp16 output, atol 1e-4*K, rtol 1e-3,
tests/test_w8a8_block_fp8_matmul.py:107) is applied to its own shape list as well."""
import os

import numpy as np
import pytest
import torch

import flag_gems
from oracle import fp8_linear_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
FP8 = torch.float8_e4m3fn
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _ref_inputs(M, N, K, seed=0):
    """Inputs as the reference test builds them (tests/test_w8a8_block_fp8_matmul.py:65-74)."""
    g = torch.Generator().manual_seed(seed)
    A = torch.randn(M, K, generator=g).to(FP8)
    B = torch.randn(N, K, generator=g).to(FP8)
    kb, nb = (K + 127) // 128, (N + 127) // 128
    As = 0.01 * torch.rand(M, kb, generator=g) + 0.005
    Bs = 0.01 * torch.rand(nb, kb, generator=g) + 0.005
    return A, B, As, Bs


def _quantized_inputs(M, N, K, seed=0):
    """Inputs as the benchmark configurations build them: X ~ N(0,1) act-quantized 1x128,
    W ~ N(0, 0.02) quantized 128x128."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (0.02 * torch.randn(N, K, generator=g)).bfloat16()
    xq, xs = O.act_quant_ref(x, 128)
    wq, ws = O.per_block_cast_to_fp8_ref(w)
    return xq, wq, xs, ws


REF_SHAPES = [(128, 256, 512), (64, 128, 128), (256, 256, 256), (83, 7748, 3884), (84, 7168, 3884),
              (300, 520, 3884), (1100, 1000, 1000)]  # K not a multiple of 128 above 128 rows


@pytest.mark.parametrize("M,N,K", REF_SHAPES)
def test_reference_shapes_fp16_reference_tolerance(M, N, K):
    A, B, As, Bs = _ref_inputs(M, N, K)
    want = O.block_fp8_matmul_dequant_ref(A, B, As, Bs, [128, 128], torch.float32, torch.float64)
    got = flag_gems.w8a8_block_fp8_matmul(A.to(DEV), B.to(DEV), As.to(DEV), Bs.to(DEV), [128, 128], output_dtype=torch.float16)
    assert got.dtype == torch.float16 and got.shape == (M, N)
    torch.testing.assert_close(got.cpu(), want.to(torch.float16), atol=1e-4 * K, rtol=1e-3)
    # and much tighter than the reference asks: fp32 accumulation error only
    torch.testing.assert_close(got.cpu().float(), want.float(), atol=2e-3, rtol=2e-3)


@pytest.mark.parametrize("M", [1, 8, 64, 200, 512])
@pytest.mark.parametrize("N,K", [(2112, 7168), (4096, 512), (1536, 1536), (7168, 2304)])
def test_quantized_linear_shapes_bf16(M, N, K):
    xq, wq, xs, ws = _quantized_inputs(M, N, K)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    got = flag_gems.w8a8_block_fp8_matmul(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    # fp32 output against the float64 oracle: only fp32 accumulation error remains
    got32 = flag_gems.w8a8_block_fp8_matmul(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128], output_dtype=torch.float32)
    torch.testing.assert_close(got32.cpu(), want, rtol=1e-4, atol=2e-4)


@pytest.mark.parametrize("M", [17, 24, 25, 32, 40, 64])
@pytest.mark.parametrize("N,K", [(24576, 1536), (28672, 4096), (14336, 4096)])
def test_few_rows_against_wide_weights(M, N, K):
    """17 ... 64 rows against weights wide enough to give every compute unit a 128 x 128 tile (or half the units one, with
    K in two ranges) leave the decode and staged-activation kernels for the four-stage tile kernel: all of them against
    the oracle, whichever kernel the planner picks for the row count."""
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=M)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    got = flag_gems.w8a8_block_fp8_matmul(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    got32 = flag_gems.w8a8_block_fp8_matmul(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128], output_dtype=torch.float32)
    torch.testing.assert_close(got32.cpu(), want, rtol=1e-4, atol=2e-4)


def test_persistent_kernel_several_rounds_ragged_edges_and_strides():
    """M > 128 with 16-byte aligned rows takes the persistent 256x256 kernel: more tiles than compute units
    (a block walks several tiles), M and N that end inside a tile (N not a multiple of 32 either),
    column-major activation scales, a weight that is a row slice, and an output written through a view."""
    M, N, K = 1100, 13400, 384  # 5 x 53 = 265 tiles
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=3)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    got = flag_gems.w8a8_block_fp8_matmul(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    # accumulate-level check against the float64 oracle: at most one bf16 rounding plus fp32 accumulation noise
    err = (got.cpu().double() - want.double()).abs()
    assert float((err / (want.double().abs() / 128 + 2e-3)).max()) < 1.0
    s_cm = xs.t().contiguous().t().to(DEV)
    big = torch.zeros(N + 77, K, dtype=FP8)
    big[40:40 + N] = wq
    got2 = flag_gems.w8a8_block_fp8_matmul(xq.to(DEV), big.to(DEV)[40:40 + N], s_cm, ws.to(DEV), [128, 128])
    assert torch.equal(got2.view(torch.int16), got.view(torch.int16))
    # the same problem twice gives the same bits
    got3 = flag_gems.w8a8_block_fp8_matmul(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    assert torch.equal(got3.view(torch.int16), got.view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(100, 520, 2048), (128, 1300, 4096), (48, 384, 8192)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_few_tiles_split_along_k(M, N, K, dtype):
    """32 < M <= 128 with a handful of 128 x 128 tiles: the tile kernel splits K over blocks and the last
    wavefront of a tile adds the partial sums in split order.  Against the oracle in every output type, and
    bit-identical on reruns."""
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=9)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=dtype)
    assert got.dtype == dtype and got.shape == (M, N)
    tol = dict(rtol=1e-4, atol=2e-4) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got.cpu().float(), want, **tol)
    for _ in range(3):
        again = flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=dtype)
        assert torch.equal(again.view(torch.int8), got.view(torch.int8))


@pytest.mark.parametrize("M,N,K", [(2048, 512, 2048), (1300, 1000, 2304), (4096, 384, 1024), (3000, 1100, 896)])
def test_tall_problems_against_narrow_weights(M, N, K):
    """More than 1024 rows but at most one 128 x 128 tile per compute unit: the four-stage tile kernel with K split
    over blocks, not the persistent kernel.  Ragged M and N, 7 and 18 K-blocks; against the oracle and bit-identical
    on reruns."""
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=23)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(*args)
    assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    for _ in range(2):
        assert torch.equal(flag_gems.w8a8_block_fp8_matmul(*args).view(torch.int16), got.view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(129, 576, 7168), (200, 1030, 4096), (256, 2048, 2048), (190, 1280, 8192), (257, 1024, 2048),
                                   (500, 260, 8192), (512, 1000, 1152), (256, 1100, 4096), (300, 4100, 512)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_129_to_512_rows_against_tiny_weights(M, N, K, dtype):
    """Weights of a few MB: the kernel of 33 to 64 rows takes the rows in three to eight equal parts in one launch (the
    last part with fewer rows), each part reading the weights again ((200, 1030, 4096), (256, 2048, 2048), (190, 1280, 8192),
    (256, 1100, 4096), (300, 4100, 512)); against the very smallest the decode kernels take sixteen or thirty-two parts
    of up to 16 rows (the others).  Ragged M and N, column-major activation scales; against the oracle and bit-identical
    on reruns."""
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=29)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=dtype)
    assert got.dtype == dtype and got.shape == (M, N)
    tol = dict(rtol=1e-4, atol=4e-4) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got.cpu().float(), want, **tol)
    for _ in range(2):
        assert torch.equal(flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=dtype).view(torch.int8), got.view(torch.int8))
    xs_cm = xs.to(DEV).t().contiguous().t()
    cm = flag_gems.w8a8_block_fp8_matmul(args[0], args[1], xs_cm, args[3], [128, 128], output_dtype=dtype)
    assert torch.equal(cm.view(torch.int8), got.view(torch.int8))


@pytest.mark.parametrize("M,N,K", [(700, 4000, 4096), (512, 6144, 4096), (1000, 3200, 8192), (300, 10000, 1024),
                                   (768, 7168, 2304), (256, 24576, 1536), (1000, 6100, 4096), (130, 40000, 512)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_129_to_512_tiles_of_128_rows(M, N, K, dtype):
    """129..256 tiles of 128 x 128 with K <= 8192: two blocks per tile, the second half's sums added in split order;
    257..512 tiles with short K: the tile kernel, one block per tile.  Ragged M and N; against the oracle and
    bit-identical on reruns."""
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=17)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=dtype)
    tol = dict(rtol=1e-4, atol=4e-4) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got.cpu().float(), want, **tol)
    for _ in range(2):
        assert torch.equal(flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=dtype).view(torch.int8), got.view(torch.int8))


@pytest.mark.parametrize("M,N,K", [(33, 100, 384), (64, 2112, 7168), (50, 7168, 16384), (40, 24584, 1536), (64, 4104, 2304),
                                   (33, 49152, 2048), (48, 20490, 1536), (37, 16384, 1024), (33, 20480, 3072),
                                   (65, 520, 1024), (100, 2112, 4096), (128, 4096, 4096), (128, 7000, 2304),
                                   (48, 8330, 6144), (64, 6650, 8192), (40, 8200, 1024), (64, 16384, 1152), (70, 16650, 8192),
                                   (64, 33040, 2048), (44, 36000, 2560),
                                   (65, 2112, 7168), (97, 1030, 8192), (128, 8200, 1024), (81, 3000, 4224), (128, 2048, 16384),
                                   (33, 512, 7168), (47, 1030, 8192), (64, 2048, 2048), (50, 8200, 1024),
                                   (40, 2112, 7168), (64, 1536, 12288), (35, 8192, 1536), (100, 1000, 8192), (128, 2048, 2048), (77, 1536, 7168)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_33_to_128_rows(M, N, K, dtype):
    """33 <= M <= 64 (and 65 <= M <= 128 with small weights) takes the kernel that keeps the activations in LDS and
    streams the weights (wide weights with up to 48 rows: a wavefront per 16 weight rows, the second line of shapes): one K range or several (partial sums added in split order), N that ends inside a 16-row
    group, fewer rows than are staged, every output type, column-major scales; against the oracle and bit-identical
    on reruns.  The last line of shapes: that kernel's blocks would leave a second round of compute units mostly idle,
    so the four-stage tile kernel takes them with K in three and four ranges; the last shape has 131 tiles, which that kernel
    splits in three ranges rather than leave half of the compute units idle; the two after it are too wide for one round of tiles
    and run in rounds of blocks whose K split is chosen by how full the rounds are; the last five (and (65, 520, 1024),
    (100, 2112, 4096), (128, 4096, 4096) above) have 65 to 128 rows against small weights, which the same kernel takes as two
    halves of the rows in one launch (48 or 64 rows staged, a second half with fewer rows than the first); the last two lines are
    33 to 64 rows against weights of up to 13 MB (26 MB when narrow), which the decode kernels take in four parts of up to 16
    rows that share rows where the count does not divide, and 65 to 128 rows against weights of up to 11.5 MB in eight parts
    ((50, 8200, 1024) is just too wide for that and stays on the staged-activation kernel)."""
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=13)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=dtype)
    assert got.dtype == dtype and got.shape == (M, N)
    tol = dict(rtol=1e-4, atol=2e-4) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got.cpu().float(), want, **tol)
    for _ in range(2):
        assert torch.equal(flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=dtype).view(torch.int8), got.view(torch.int8))
    xs_cm = xs.to(DEV).t().contiguous().t()
    cm = flag_gems.w8a8_block_fp8_matmul(args[0], args[1], xs_cm, args[3], [128, 128], output_dtype=dtype)
    assert torch.equal(cm.view(torch.int8), got.view(torch.int8))


@pytest.mark.parametrize("M,N,K", [(1, 2112, 7168), (16, 2112, 7168), (5, 1000, 7168), (3, 200, 8192), (7, 300, 16512),
                                   (16, 4608, 7168), (12, 7168, 16384), (2, 7168, 16384), (1, 24576, 1536),
                                   (32, 2112, 7168), (20, 4608, 4096), (1, 9, 1024), (4, 130, 2048), (9, 4099, 7296),
                                   (16, 32768, 512), (5, 24580, 384), (2, 20480, 256), (16, 28672, 4096),
                                   (16, 4612, 7296), (13, 7168, 16512), (16, 8192, 8192), (10, 5000, 12416), (8, 7168, 16384),
                                   (17, 24576, 1536), (32, 32768, 512), (24, 20490, 640), (31, 49152, 1024), (32, 24584, 1536),
                                   (19, 20480, 256), (32, 28672, 4096), (24, 20488, 3072), (32, 32768, 2048),
                                   (24, 16384, 1024), (17, 16400, 2048), (16, 18432, 1024), (3, 17416, 1536),
                                   (16, 2304, 16384), (9, 3590, 18944), (12, 4096, 11008), (16, 1280, 8192), (16, 1000, 8192),
                                   (8, 2050, 16384), (24, 8192, 1024), (17, 2050, 1152),
                                   (17, 2304, 16384), (32, 3590, 18944), (24, 4096, 14336),
                                   (21, 2112, 7168), (32, 4608, 7168), (30, 4100, 4096), (25, 5000, 7296), (20, 2112, 7168),
                                   (9, 4096, 14336)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_up_to_32_rows_uneven_chunks(M, N, K, dtype):
    """M <= 32 takes the kernel that deals the weight rows out evenly over the compute units: chunks that differ by a
    row and begin anywhere (so that a chunk's rows lie in two 128-row scale blocks), chunks of fewer than 16 rows, N
    that is no multiple of 4, K split over blocks, an odd number of K-blocks, activations kept in LDS (long K, M <=
    16) or fetched per K-block (short K, M > 16), wide weights (a wavefront per 16 rows, the four shapes from
    (16, 32768, 512) on: K of 2, 3 and 4 K-blocks, N that ends inside a 16-row group, activations that eight wavefronts share),
    activations too large for LDS as a whole and copied pair by pair into two slots per wavefront (M = 12 with
    K = 16384 and the five shapes from (16, 4612, 7296) on: an odd number of K-blocks, chunks that begin anywhere), wide
    weights with 17 to 32 rows (the block shares two 16-row images of the activations; the shapes from (17, 24576, 1536) on, of which
    (32, 28672, 4096) is too long in K for that and stays on the kernels for 32 rows, two take blocks of eight
    wavefronts, and the four up to (3, 17416, 1536) have just over four 16-row groups per compute unit), narrow weights
    with 128 KB of activations or more (half the blocks on half of K each, the half ranges in LDS or in the two slots;
    the six shapes from (16, 2304, 16384) on and (9, 4096, 14336)), 17 to 32 rows against short K and few tiles
    ((24, 8192, 1024) and the next), 17 to 32 rows against weights of up to 6144 rows (two parts of up to 16 rows in one
    launch, sharing the middle row when the count is odd: (20, 4608, 4096), (17, 2050, 1152), the three from
    (17, 2304, 16384) on and the five from (21, 2112, 7168) on), column-major activation scales; against the oracle and
    bit-identical on reruns."""
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=17)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=dtype)
    assert got.dtype == dtype and got.shape == (M, N)
    tol = dict(rtol=1e-4, atol=2e-4) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got.cpu().float(), want, **tol)
    for _ in range(2):
        assert torch.equal(flag_gems.w8a8_block_fp8_matmul(*args, output_dtype=dtype).view(torch.int8), got.view(torch.int8))
    xs_cm = xs.to(DEV).t().contiguous().t()
    cm = flag_gems.w8a8_block_fp8_matmul(args[0], args[1], xs_cm, args[3], [128, 128], output_dtype=dtype)
    assert torch.equal(cm.view(torch.int8), got.view(torch.int8))


@pytest.mark.parametrize("N,K", [(2112, 7168), (4608, 7168)])
def test_rows_of_a_small_batch_do_not_depend_on_its_size(N, K):
    """Row m of the product is the same bits whether the call has 1, 8 or 16 activation rows: the kernels for M <= 16
    differ only in where the activations are kept (all of them in LDS, or two slots per wavefront refilled pair by
    pair: N = 4608 with 16 rows)."""
    xq, wq, xs, ws = _quantized_inputs(16, N, K, seed=23)
    xq, wq, xs, ws = xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV)
    full = flag_gems.w8a8_block_fp8_matmul(xq, wq, xs, ws, [128, 128], output_dtype=torch.float32)
    for rows in (1, 8):
        part = flag_gems.w8a8_block_fp8_matmul(xq[:rows].contiguous(), wq, xs[:rows].contiguous(), ws, [128, 128], output_dtype=torch.float32)
        assert torch.equal(part.view(torch.int32), full[:rows].view(torch.int32))


@pytest.mark.parametrize("M,N,K", [(1024, 7168, 8192), (300, 7000, 16384)])
def test_tiles_cut_into_equal_ranges_along_k(M, N, K):
    """112 tiles x 64 K-blocks and 56 tiles x 128 K-blocks (ragged in M and N): the persistent kernel cuts every
    tile into ranges of at least 32 K-blocks that fill most of the GPU, one block per range, and the last
    wavefront to arrive adds the ranges' partial sums in range order.  Against the oracle, and bit-identical on
    reruns."""
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=11)
    want = O.block_fp8_matmul_tiled_ref(xq, wq, xs, ws, [128, 128], torch.float32)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(*args)
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    err = (got.cpu().double() - want.double()).abs()
    assert float((err / (want.double().abs() / 128 + 2e-3)).max()) < 1.0
    for _ in range(3):
        assert torch.equal(flag_gems.w8a8_block_fp8_matmul(*args), got)


@pytest.mark.parametrize("M,N,K", [(2304, 8192, 8192), (2250, 8104, 8192)])
def test_whole_rounds_then_the_last_tiles_shared(M, N, K):
    """288 tiles on 256 compute units: one launch computes 256 whole tiles, a second one cuts the other 32 into 4
    ranges each so that half of the units take part (aligned and ragged shapes).  Against the oracle, bit-identical
    on reruns."""
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=17)
    want = O.block_fp8_matmul_tiled_ref(xq, wq, xs, ws, [128, 128], torch.float32)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(*args)
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    err = (got.cpu().double() - want.double()).abs()
    assert float((err / (want.double().abs() / 128 + 2e-3)).max()) < 1.0
    for _ in range(2):
        assert torch.equal(flag_gems.w8a8_block_fp8_matmul(*args), got)


@pytest.mark.parametrize("M,N,K", [(1100, 1300, 8192), (1200, 3000, 4096)])
def test_activation_scales_in_either_layout_give_the_same_bits(M, N, K):
    """The persistent kernel reads activation scales K-block by K-block for 64 rows at a time.  Row-major
    scales ([M, K/128] contiguous, what the quantizer returns) are first transposed into the workspace;
    scales that already have the rows contiguous (strides (1, M), the reference's column_major_scales
    layout) are read in place; a call without workspace reads the row-major ones as they are.  All three
    The first two run the same kernel on the same values and must agree bit for bit; the call without
    workspace may also add the K-blocks in another order (no tile is shared between blocks then)."""
    from flaggems_amd import _lib
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=5)
    xq, wq, xs, ws = xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV)
    want = O.block_fp8_matmul_dequant_ref(xq.cpu(), wq.cpu(), xs.cpu(), ws.cpu(), [128, 128], torch.float32, torch.float64)
    got = flag_gems.w8a8_block_fp8_matmul(xq, wq, xs, ws, [128, 128])
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    xs_cm = xs.t().contiguous().t()
    assert xs_cm.stride() == (1, M)
    got_cm = flag_gems.w8a8_block_fp8_matmul(xq, wq, xs_cm, ws, [128, 128])
    assert torch.equal(got_cm.view(torch.int16), got.view(torch.int16))
    lib = _lib.load()
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    status = lib.fg_block_fp8_gemm(xq.data_ptr(), K, wq.data_ptr(), K, xs.data_ptr(), xs.stride(0), xs.stride(1),
                                   ws.data_ptr(), ws.stride(0), ws.stride(1), out.data_ptr(), N, _lib.DTYPE_CODE[torch.bfloat16],
                                   M, N, K, 128, 128, None, 0, _lib.current_stream_ptr(torch.device(DEV)))
    _lib.check(status, "fg_block_fp8_gemm")
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu().float(), want, rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(out.float(), got.float(), rtol=8e-3, atol=1e-3)  # one bf16 ulp


def test_tiles_split_along_k_between_blocks():
    """18 tiles of 64 K-blocks on a 256-unit GPU: the persistent kernel cuts the 1152 steps into contiguous
    ranges, so every tile is computed by many blocks and finished through the workspace.  Ragged M and N,
    results against the oracle, and bit-identical on a second run (partial sums are added in a fixed order)."""
    M, N, K = 700, 1300, 8192
    from flaggems_amd import _lib
    lib = _lib.load()
    xq, wq, xs, ws = _quantized_inputs(M, N, K, seed=11)
    want = O.block_fp8_matmul_dequant_ref(xq, wq, xs, ws, [128, 128], torch.float32, torch.float64)
    args = (xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), [128, 128])
    got = flag_gems.w8a8_block_fp8_matmul(*args)
    torch.testing.assert_close(got.cpu().float(), want, rtol=1e-2, atol=1e-2)
    err = (got.cpu().double() - want.double()).abs()
    assert float((err / (want.double().abs() / 128 + 2e-3)).max()) < 1.0
    for _ in range(3):
        again = flag_gems.w8a8_block_fp8_matmul(*args)
        assert torch.equal(again.view(torch.int16), got.view(torch.int16))
    # the shape is one the library wants a workspace for; without one (C ABI called directly) whole tiles
    # go to the blocks and the result differs at most by fp32 summation order
    assert lib.fg_block_fp8_gemm_workspace_bytes(M, N, K) > 16384
    a, b, s_a, s_b = args[:4]
    c = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    rc = lib.fg_block_fp8_gemm(a.data_ptr(), K, b.data_ptr(), K, s_a.data_ptr(), s_a.stride(0), s_a.stride(1),
                               s_b.data_ptr(), s_b.stride(0), s_b.stride(1), c.data_ptr(), N, _lib.DTYPE_CODE[torch.bfloat16],
                               M, N, K, 128, 128, None, 0, _lib.current_stream_ptr(torch.device(DEV)))
    assert rc == 0
    torch.testing.assert_close(c.cpu().float(), want, rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(c.float(), got.float(), rtol=8e-3, atol=1e-3)


def test_closed_forms():
    A, B, As, Bs = _ref_inputs(48, 384, 512, seed=3)
    # unit scales -> plain matmul, exact in fp32 for these magnitudes up to summation order
    got = flag_gems.w8a8_block_fp8_matmul(A.to(DEV), B.to(DEV), torch.ones_like(As).to(DEV), torch.ones_like(Bs).to(DEV), [128, 128], output_dtype=torch.float32)
    # the fp8 MFMA sums the 128 products of a K-block with about 14 bits below the largest product
    # (measured on MI355X: 448 + 448*2^-14 -> 448), so the bound is relative to sum |a||b|
    bound = 1e-3 * (A.float().abs() @ B.float().abs().T)
    assert ((got.cpu() - A.float() @ B.float().T).abs() <= bound + 1e-6).all()
    # one-hot rows pick single scaled weight entries exactly
    cols = [0, 127, 128, 511]
    a = torch.zeros(48, 512)
    for r in range(48):
        a[r, cols[r % 4]] = 1.0
    got = flag_gems.w8a8_block_fp8_matmul(a.to(FP8).to(DEV), B.to(DEV), As.to(DEV), Bs.to(DEV), [128, 128], output_dtype=torch.float32).cpu()
    for r in range(48):
        c = cols[r % 4]
        want = B[:, c].float() * As[r, c // 128] * Bs[:, c // 128].repeat_interleave(128)[:384]
        torch.testing.assert_close(got[r], want, rtol=1e-6, atol=0)
    # K-block-specific power-of-two scales are applied to the right block, exactly
    as2 = torch.tensor([[2.0, 0.5, 4.0, 0.25]]).repeat(48, 1)
    bs2 = torch.tensor([[0.25, 4.0, 1.0, 8.0]]).repeat(3, 1)
    got = flag_gems.w8a8_block_fp8_matmul(A.to(DEV), B.to(DEV), as2.to(DEV), bs2.to(DEV), [128, 128], output_dtype=torch.float32).cpu()
    af, bf = A.float(), B.float()
    want = sum((af[:, i * 128:(i + 1) * 128] @ bf[:, i * 128:(i + 1) * 128].T) * float(as2[0, i] * bs2[0, i]) for i in range(4))
    assert ((got - want).abs() <= 1e-3 * sum((af[:, i * 128:(i + 1) * 128].abs() @ bf[:, i * 128:(i + 1) * 128].abs().T) * float(as2[0, i] * bs2[0, i]) for i in range(4))).all()


def test_leading_dims_strided_scales_and_fp8_matmul_alias():
    xq, wq, xs, ws = _quantized_inputs(24, 640, 1024, seed=5)
    want = O.block_fp8_matmul_tiled_ref(xq, wq, xs, ws, [128, 128], torch.float32)
    a = xq.view(2, 3, 4, 1024).to(DEV)
    s = xs.view(2, 3, 4, 8).to(DEV)
    got = flag_gems.w8a8_block_fp8_matmul(a, wq.to(DEV), s, ws.to(DEV), [128, 128])
    assert got.shape == (2, 3, 4, 640)
    torch.testing.assert_close(got.view(24, 640).cpu().float(), want, rtol=1e-2, atol=1e-2)
    # column-major activation scales (strides (1, M)) and a weight that is a row-slice of a bigger one
    s_cm = xs.t().contiguous().t().to(DEV)
    big = torch.zeros(700, 1024, dtype=FP8)
    big[30:670] = wq
    got2 = flag_gems.w8a8_block_fp8_matmul(xq.to(DEV), big.to(DEV)[30:670], s_cm, ws.to(DEV), [128, 128])
    assert torch.equal(got2.view(torch.int16), got.view(24, 640).view(torch.int16))
    got3 = flag_gems.fp8_matmul(a, s, wq.to(DEV), ws.to(DEV))
    assert got3.shape == (2, 3, 4, 640) and got3.dtype == torch.bfloat16
    assert torch.equal(got3.view(torch.int16), got.view(torch.int16))


def test_config1_golden():
    z = np.load(os.path.join(GOLD, "config1.npz"))
    x, w = O.make_config1(0)
    xq, xs = flag_gems.act_quant_triton(x.to(DEV), 128)
    wq, ws = O.per_block_cast_to_fp8_ref(w)
    c = flag_gems.w8a8_block_fp8_matmul(xq, wq.to(DEV), xs, ws.to(DEV), [128, 128])
    want = torch.from_numpy(z["c_bits"]).view(torch.bfloat16)
    assert c.shape == (64, 512)
    torch.testing.assert_close(c.cpu().float(), want.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("N,K", [(2112, 7168), (24576, 1536), (32768, 512), (7168, 16384), (4608, 7168), (7168, 2304)])
def test_full_size_linearity_and_row_consistency(N, K):
    """M = 4096 DeepSeek-V3 shapes: properties that need no CPU matmul.
    (1) rows are independent: the first 8 rows equal an M=8 call (compared with the oracle);
    (2) doubling one K-block's activation scale adds exactly that block's contribution."""
    M = 4096
    g = torch.Generator(device=DEV).manual_seed(0)
    A = torch.randn(M, K, device=DEV, generator=g).to(FP8)
    B = (torch.randn(N, K, device=DEV, generator=g)).to(FP8)
    As = 0.01 * torch.rand(M, K // 128, device=DEV, generator=g) + 0.005
    Bs = 0.01 * torch.rand((N + 127) // 128, K // 128, device=DEV, generator=g) + 0.005
    C = flag_gems.w8a8_block_fp8_matmul(A, B, As, Bs, [128, 128], output_dtype=torch.float32)
    rows = torch.tensor([0, 1, 255, 256, 2047, 4095], device=DEV)
    want = O.block_fp8_matmul_dequant_ref(A[rows].cpu(), B.cpu(), As[rows].cpu(), Bs.cpu(), [128, 128], torch.float32, torch.float64)
    torch.testing.assert_close(C[rows].cpu(), want, rtol=1e-4, atol=1e-4)
    As2 = As.clone()
    As2[:, 1] *= 2
    C2 = flag_gems.w8a8_block_fp8_matmul(A, B, As2, Bs, [128, 128], output_dtype=torch.float32)
    only1 = torch.zeros_like(As)
    only1[:, 1] = As[:, 1]
    C1 = flag_gems.w8a8_block_fp8_matmul(A, B, only1, Bs, [128, 128], output_dtype=torch.float32)
    torch.testing.assert_close(C2 - C, C1, rtol=1e-3, atol=1e-4)


def test_host_side_assertions():
    A, B, As, Bs = (t.to(DEV) for t in _ref_inputs(16, 256, 256))
    with pytest.raises(AssertionError):
        flag_gems.w8a8_block_fp8_matmul(A, B[:, :128], As, Bs, [128, 128])
    with pytest.raises(AssertionError):
        flag_gems.w8a8_block_fp8_matmul(A, B, As[:, :1], Bs, [128, 128])
    with pytest.raises(AssertionError):
        flag_gems.w8a8_block_fp8_matmul(A.t(), B, As, Bs, [128, 128])
    out = flag_gems.w8a8_block_fp8_matmul(A[:0], B, As[:0], Bs, [128, 128])
    assert out.shape == (0, 256)


@pytest.mark.parametrize("block_size", [[256, 128], [128, 256], [256, 256], [384, 512]])
@pytest.mark.parametrize("M,N,K", [(7, 640, 1024), (100, 1000, 1536), (300, 2304, 4096), (4096, 2112, 7168)])
def test_scale_blocks_that_are_multiples_of_128(M, N, K, block_size):
    """block_size other than [128, 128] (the reference's kernel takes any: src/flag_gems/ops/w8a8_block_fp8_matmul.py:
    173-232): blocks of whole multiples of 128, ragged at the edges of N and K, against the oracle evaluated with the
    same block_size."""
    block_n, block_k = block_size
    g = torch.Generator().manual_seed(M + N + K + block_n)
    A = torch.randn(M, K, generator=g).to(FP8)
    B = torch.randn(N, K, generator=g).to(FP8)
    As = 0.01 * torch.rand(M, -(-K // block_k), generator=g) + 0.005
    Bs = 0.01 * torch.rand(-(-N // block_n), -(-K // block_k), generator=g) + 0.005
    got = flag_gems.w8a8_block_fp8_matmul(A.to(DEV), B.to(DEV), As.to(DEV), Bs.to(DEV), block_size).cpu().float()
    rows = torch.arange(M) if M <= 300 else torch.tensor([0, 1, 255, 256, 257, M // 2, M - 1])
    want = O.block_fp8_matmul_dequant_ref(A[rows], B, As[rows], Bs, block_size, torch.float32, torch.float64)
    torch.testing.assert_close(got[rows], want, rtol=1e-2, atol=1e-2)
    # and the bits of the call with the scales written out per 128 x 128 block
    As128 = As.repeat_interleave(block_k // 128, dim=1)[:, : -(-K // 128)].contiguous()
    Bs128 = Bs.repeat_interleave(block_n // 128, dim=0)[: -(-N // 128)].repeat_interleave(block_k // 128, dim=1)[:, : -(-K // 128)].contiguous()
    same = flag_gems.w8a8_block_fp8_matmul(A.to(DEV), B.to(DEV), As128.to(DEV), Bs128.to(DEV), [128, 128]).cpu().float()
    assert torch.equal(same, got)


@pytest.mark.parametrize("block_size", [[64, 64], [64, 128], [128, 64], [32, 96], [100, 60], [128, 200], [1, 7], [4096, 32]])
@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (7, 640, 1000), (100, 1000, 1536), (300, 2112, 4096), (2100, 330, 777), (130, 200, 1008)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_scale_blocks_of_any_size(M, N, K, block_size, dtype):
    """block_size that is no multiple of 128 (64-wide groups, blocks that divide nothing, a block wider than N, a
    K-group of 7): the tile kernel on the 16x16x32 matrix instruction where block_k is a multiple of 32, block_n of 16
    and K of 16, the plain kernel otherwise, against the oracle evaluated with the same block_size; M, N and K that
    end inside the tiles and K rounds of both."""
    block_n, block_k = block_size
    if dtype == torch.float32 and (M, N, K) not in ((7, 640, 1000), (2100, 330, 777), (130, 200, 1008)):
        pytest.skip("fp32 output on two shapes")
    g = torch.Generator().manual_seed(M + N + K + block_n + block_k)
    A = torch.randn(M, K, generator=g).to(FP8)
    B = torch.randn(N, K, generator=g).to(FP8)
    As = 0.01 * torch.rand(M, -(-K // block_k), generator=g) + 0.005
    Bs = 0.01 * torch.rand(-(-N // block_n), -(-K // block_k), generator=g) + 0.005
    got = flag_gems.w8a8_block_fp8_matmul(A.to(DEV), B.to(DEV), As.to(DEV), Bs.to(DEV), block_size, output_dtype=dtype)
    assert got.dtype == dtype and got.shape == (M, N)
    want = O.block_fp8_matmul_dequant_ref(A, B, As, Bs, block_size, torch.float32, torch.float64)
    tol = dict(rtol=1e-4, atol=2e-4) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got.cpu().float(), want, **tol)
    # strided scales (column-major activation scales) give the same bits
    as_cm = As.to(DEV).t().contiguous().t()
    again = flag_gems.w8a8_block_fp8_matmul(A.to(DEV), B.to(DEV), as_cm, Bs.to(DEV), block_size, output_dtype=dtype)
    assert torch.equal(again.view(torch.int8), got.view(torch.int8))


@pytest.mark.parametrize("rows,stride,parts,N,K", [(9, 8, 2, 2112, 7168), (16, 15, 2, 6144, 4096), (11, 8, 4, 2112, 7168),
                                                    (16, 13, 4, 8192, 1536), (13, 9, 8, 1536, 7168), (9, 8, 16, 512, 7168),
                                                    (16, 11, 32, 1024, 2048)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_parts_that_share_rows_agree_bit_for_bit(rows, stride, parts, N, K, dtype):
    """17 to 512 rows against small weights run as 2, 4, 8 ... parts of up to 16 rows, the entries of a batch that shares
    the weights, and the last part starts early so that it ends with the last row: the rows it shares with the part
    before are computed, and stored, by both.  That is safe because a row's result depends neither on the entry that
    computes it nor on its place within the entry: here a batch of such entries, `stride` < `rows` rows apart, goes
    through the C ABI with a buffer per entry, and the rows that neighbours share come out with equal bits (bf16 and
    fp32, K in one range and split over blocks)."""
    from flaggems_amd import _lib
    lib = _lib.load()
    M = (parts - 1) * stride + rows
    xq, wq, xs, ws = (t.to(DEV) for t in _quantized_inputs(M, N, K, seed=31))
    kb = K // 128
    c = torch.zeros(parts, rows, N, dtype=dtype, device=DEV)
    need = lib.fg_batched_block_fp8_gemm_workspace_bytes(parts, rows, N, K)
    wsp = _lib.workspace(torch.device(DEV), need) if need else None
    rc = lib.fg_batched_block_fp8_gemm(
        xq.data_ptr(), K, stride * K, wq.data_ptr(), K, 0, xs.data_ptr(), kb, 1, stride * kb, ws.data_ptr(), kb, 1, 0,
        c.data_ptr(), N, rows * N, _lib.DTYPE_CODE[dtype], parts, rows, N, K, 128, 128,
        wsp.data_ptr() if need else None, wsp.numel() if need else 0, _lib.current_stream_ptr(torch.device(DEV)))
    _lib.check(rc, "fg_batched_block_fp8_gemm")
    torch.cuda.synchronize()
    want = O.block_fp8_matmul_dequant_ref(xq.cpu(), wq.cpu(), xs.cpu(), ws.cpu(), [128, 128], torch.float32, torch.float64)
    tol = dict(rtol=1e-4, atol=4e-4) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    shared = rows - stride
    for z in range(parts):
        torch.testing.assert_close(c[z].cpu().float(), want[z * stride:z * stride + rows], **tol)
        if z + 1 < parts:
            assert torch.equal(c[z][stride:].view(torch.int8), c[z + 1][:shared].view(torch.int8))
