// Block-scaled FP8 GEMM for scale blocks of any size: C[m, n] = sum over K-groups g of
//   ( sum_{k in group g} A[m, k] * B[n, k] ) * As[m, g] * Bs[n / block_n, g],      group g = k / block_k.
//
// The reference's kernel takes any block_size = [block_n, block_k]
// (src/flag_gems/ops/w8a8_block_fp8_matmul.py:51-122, 173-232); the matrix-instruction kernels of this library apply
// one scale product per 128-wide K-block and serve 128 x 128 blocks (and, through the host, their multiples).  This
// kernel is the path for everything else -- 64-wide groups, blocks that divide nothing -- so that no block_size is
// refused.  It is a plain tiled fp32 kernel, not a fast one: a 64 x 64 tile per workgroup, operands widened to fp32
// on their way into LDS, 4 x 4 results per thread; the products of a K-group are summed in fp32 and enter the result
// times the two scales when the group ends, the order in which the reference's kernel does it
// (w8a8_block_fp8_matmul.py:108-117: accumulator += dot(a, b) * a_s[:, None] * b_s[None, :]).
// Measured: M = 4096, N = 2112, K = 7168 with 64 x 64 blocks in 4.1 ms (30 TFLOP/s; 78 us with 128 x 128 blocks on the
// matrix-instruction kernel).

#include "fp8_gemm_common.h"

namespace fg {
namespace {

constexpr int kAnyTile = 64;    // rows and columns of a workgroup's tile
constexpr int kAnyChunk = 32;   // K elements staged per round
constexpr int kAnyPad = 4;      // floats of padding per staged row of 64: rows 68 floats apart

struct AnyBlockArgs {
  GemmArgs g;
  int block_n, block_k;
};

__global__ __launch_bounds__(256) void block_fp8_gemm_anyblock_kernel(AnyBlockArgs a) {
  __shared__ float xs_lds[kAnyChunk][kAnyTile + kAnyPad];  // [k][m]
  __shared__ float ws_lds[kAnyChunk][kAnyTile + kAnyPad];  // [k][n]
  const GemmArgs& g = a.g;
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;           // 4 columns at tx * 4, 4 rows at ty * 4
  const int m0 = blockIdx.y * kAnyTile, n0 = blockIdx.x * kAnyTile;
  // staging: thread -> row tid / 4 of the tile, 8 consecutive k at (tid % 4) * 8
  const int srow = tid >> 2, sk = (tid & 3) * 8;
  const int xm = m0 + srow, wn = n0 + srow;
  const uint8_t* const xrow = g.X + (int64_t)(xm < g.M ? xm : g.M - 1) * g.ldx;
  const uint8_t* const wrow = g.W + (int64_t)(wn < g.N ? wn : g.N - 1) * g.ldw;

  float acc[4][4], part[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) { acc[i][j] = 0.f; part[i][j] = 0.f; }
  // rows and scale-block columns of this thread's results (clamped: results outside the matrix are not stored)
  int rows[4], nblk[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + i;
    rows[i] = m < g.M ? m : g.M - 1;
    nblk[i] = (n < g.N ? n : g.N - 1) / a.block_n;
  }

  for (int k0 = 0; k0 < g.K; k0 += kAnyChunk) {
    // byte loads: K and the row strides may be anything
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int k = k0 + sk + e;
      const bool in = k < g.K;
      const int xb = in ? xrow[k] : 0, wb = in ? wrow[k] : 0;
      xs_lds[sk + e][srow] = __builtin_amdgcn_cvt_f32_fp8(xb, 0);
      ws_lds[sk + e][srow] = __builtin_amdgcn_cvt_f32_fp8(wb, 0);
    }
    __syncthreads();
    const int chunk = g.K - k0 < kAnyChunk ? g.K - k0 : kAnyChunk;
    for (int kk = 0; kk < chunk; ++kk) {
      const v4f xv = *reinterpret_cast<const v4f*>(&xs_lds[kk][ty * 4]);
      const v4f wv = *reinterpret_cast<const v4f*>(&ws_lds[kk][tx * 4]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = __builtin_fmaf(xv[i], wv[j], part[i][j]);
      const int k = k0 + kk;
      if ((k + 1) % a.block_k == 0 || k + 1 == g.K) {  // uniform: the K-group ends here
        const int kg = k / a.block_k;
        float sx[4], sw[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          sx[i] = g.xs[(int64_t)rows[i] * g.xs_rs + (int64_t)kg * g.xs_cs];
          sw[i] = g.ws[(int64_t)nblk[i] * g.ws_rs + (int64_t)kg * g.ws_cs];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            acc[i][j] = acc[i][j] + (part[i][j] * sx[i]) * sw[j];
            part[i][j] = 0.f;
          }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < g.M && n < g.N) store_output<kModeBlock>(g, m, n, acc[i][j]);
    }
}

}  // namespace

int launch_anyblock(const GemmArgs& g, int64_t block_n, int64_t block_k, hipStream_t stream) {
  if (block_n < 1 || block_k < 1 || block_n > 0x7FFFFFFF || block_k > 0x7FFFFFFF)
    FG_FAIL(FG_ERR_INVALID_ARG, "block fp8 gemm: scale block %lld x %lld", (long long)block_n, (long long)block_k);
  const int64_t tiles_n = ceil_div((int64_t)g.N, (int64_t)kAnyTile), tiles_m = ceil_div((int64_t)g.M, (int64_t)kAnyTile);
  if (tiles_m > 65535) FG_FAIL(FG_ERR_UNSUPPORTED, "block fp8 gemm with %lld x %lld scale blocks: more than %d rows", (long long)block_n,
                               (long long)block_k, 65535 * kAnyTile);
  AnyBlockArgs a;
  a.g = g;
  a.block_n = (int)block_n;
  a.block_k = (int)block_k;
  FG_LAUNCH(block_fp8_gemm_anyblock_kernel, dim3((uint32_t)tiles_n, (uint32_t)tiles_m), dim3(256), 0, stream, a);
  FG_CHECK_LAUNCH("block_fp8_gemm_anyblock_kernel");
  return FG_OK;
}

}  // namespace fg
