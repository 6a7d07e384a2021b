// Block-scaled FP8 GEMM for scale blocks of any size: C[m, n] = sum over K-groups g of
//   ( sum_{k in group g} A[m, k] * B[n, k] ) * As[m, g] * Bs[n / block_n, g],      group g = k / block_k.
//
// The reference's kernel takes any block_size = [block_n, block_k]
// (src/flag_gems/ops/w8a8_block_fp8_matmul.py:51-122, 173-232); the matrix-instruction kernels of this library apply
// one scale product per 128-wide K-block and serve 128 x 128 blocks (and, through the host, their multiples).  This
// file is the path for everything else -- 64-wide groups, blocks that divide nothing -- so that no block_size is
// refused.  Two kernels, both summing the products of a K-group in fp32 and adding them to the result times the two
// scales when the group ends, the order in which the reference's kernel does it
// (w8a8_block_fp8_matmul.py:108-117: accumulator += dot(a, b) * a_s[:, None] * b_s[None, :]):
//   block_fp8_gemm_subblock_kernel  block_k a multiple of 32 and block_n of 16 (64 x 64, 128 x 64, 32 x 96 ...), K a multiple
//       of 16, 16-byte aligned rows: 128 x 128 tiles through LDS and v_mfma_f32_16x16x32_fp8_fp8, whose 32 elements of K
//       never straddle a group.
//   block_fp8_gemm_anyblock_kernel  anything: a plain tiled fp32 kernel, a 64 x 64 tile per workgroup, operands widened
//       to fp32 on their way into LDS, 4 x 4 results per thread.
// Measured, M = 4096, N = 2112, K = 7168 with 64 x 64 blocks: 4.1 ms on the plain kernel (30 TFLOP/s), 0.36 ms on the
// matrix-instruction one (343 TFLOP/s; 64 x 128 blocks 0.27 ms; M = N = K = 4096: 530 and 742 TFLOP/s); 128 x 128 blocks
// take 0.09 ms on the kernels built for them.

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

// ---- scale blocks of 32 k x 16 n granularity on the matrix cores
constexpr int kSubTile = 128;                         // rows and columns of C per workgroup
constexpr int kSubRowBytes = 128;                     // K bytes staged per step
constexpr int kSubPanelBytes = kSubTile * kSubRowBytes;   // 16 KB
constexpr int kSubThreads = 256;
constexpr int kSubChunks = kSubTile * (kSubRowBytes / 16) / kSubThreads;  // 16-byte chunks per thread and panel: 4

__device__ __forceinline__ int sub_chunk_offset(int row, int chunk) { return row * kSubRowBytes + ((chunk ^ (row & 7)) << 4); }

// Four wavefronts, 64 x 64 results each as 4 x 4 MFMA tiles; the weights take the first operand slot, so a lane holds
// four consecutive columns n = 16 j + 4 (lane / 16) + e of row m = 16 i + lane % 16, and a 16-column tile lies inside one
// scale block.  Per step the 256 threads copy the 128 x 128-byte panels of both operands into one of two LDS stages
// (chunks XORed with the row as in the other LDS kernels; bytes past K are zeros), the next step's global loads in
// flight during the MFMAs; one barrier per step.
__global__ __launch_bounds__(kSubThreads) void block_fp8_gemm_subblock_kernel(AnyBlockArgs a) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[2][2][kSubPanelBytes];  // [stage][X or W][panel]
  const GemmArgs& g = a.g;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int bm0 = blockIdx.y * kSubTile, bn0 = blockIdx.x * kSubTile;

  const int cc = tid & 7, cr = tid >> 3;  // copy duty: chunk column cc of rows cr + 32 i
  const uint8_t* xg[kSubChunks];
  const uint8_t* wg[kSubChunks];
  int lo[kSubChunks];
#pragma unroll
  for (int i = 0; i < kSubChunks; ++i) {
    const int row = cr + 32 * i;
    xg[i] = g.X + (int64_t)min(bm0 + row, g.M - 1) * g.ldx + cc * 16;
    wg[i] = g.W + (int64_t)min(bn0 + row, g.N - 1) * g.ldw + cc * 16;
    lo[i] = sub_chunk_offset(row, cc);
  }
  const u32x4 zero = {0u, 0u, 0u, 0u};
  u32x4 rx[kSubChunks], rw[kSubChunks];
  // K is a multiple of 16: a chunk lies wholly inside or wholly outside the row
  auto fetch = [&](int k) {
    const bool inside = k + cc * 16 < g.K;
#pragma unroll
    for (int i = 0; i < kSubChunks; ++i) {
      rx[i] = inside ? *reinterpret_cast<const u32x4*>(xg[i] + k) : zero;
      rw[i] = inside ? *reinterpret_cast<const u32x4*>(wg[i] + k) : zero;
    }
  };
  auto stash = [&](int stage) {
#pragma unroll
    for (int i = 0; i < kSubChunks; ++i) {
      *reinterpret_cast<u32x4*>(&lds[stage][0][lo[i]]) = rx[i];
      *reinterpret_cast<u32x4*>(&lds[stage][1][lo[i]]) = rw[i];
    }
  };

  const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;  // inside the tile
  const int r = lane & 15, q = lane >> 4;
  v4f acc[4][4], part[4][4];  // [i: 16 rows of m][j: 16 columns of n]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) { acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f}; part[i][j] = v4f{0.f, 0.f, 0.f, 0.f}; }
  // scales of this lane's rows and column tiles (clamped: results outside the matrix are not stored)
  int64_t xs_row[4], ws_row[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    xs_row[i] = (int64_t)min(bm0 + wm0 + 16 * i + r, g.M - 1) * g.xs_rs;
    ws_row[i] = (int64_t)(min(bn0 + wn0 + 16 * i, g.N - 1) / a.block_n) * g.ws_rs;
  }

  fetch(0);
  stash(0);
  __syncthreads();
  int stage = 0;
  for (int k = 0; k < g.K; k += kSubRowBytes, stage ^= 1) {
    const bool more = k + kSubRowBytes < g.K;  // uniform over the workgroup
    if (more) fetch(k + kSubRowBytes);
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) {  // 32 elements of K each
      const int k0 = k + 32 * sub;
      if (k0 < g.K) {  // uniform
        long fx[4], fw[4];
        const int chunk = 2 * sub + (q >> 1), within = (q & 1) * 8;
#pragma unroll
        for (int f = 0; f < 4; ++f) {
          fx[f] = *reinterpret_cast<const long*>(&lds[stage][0][sub_chunk_offset(wm0 + 16 * f + r, chunk) + within]);
          fw[f] = *reinterpret_cast<const long*>(&lds[stage][1][sub_chunk_offset(wn0 + 16 * f + r, chunk) + within]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) part[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(fw[j], fx[i], part[i][j], 0, 0, 0);
        if ((k0 + 32) % a.block_k == 0 || k0 + 32 >= g.K) {  // uniform: the K-group ends with these 32 elements
          const int64_t kg = k0 / a.block_k;
          float sx[4], sw[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            sx[i] = g.xs[xs_row[i] + kg * g.xs_cs];
            sw[i] = g.ws[ws_row[i] + kg * g.ws_cs];
          }
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[i][j][e] = acc[i][j][e] + (part[i][j][e] * sx[i]) * sw[j];
              part[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
            }
        }
      }
    }
    if (more) stash(stage ^ 1);
    __syncthreads();  // the other stage is complete, and every read of this one is done before it is written again
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = bm0 + wm0 + 16 * i + r;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int n = bn0 + wn0 + 16 * j + 4 * q + e;
        if (n < g.N) store_output<kModeBlock>(g, m, n, acc[i][j][e]);
      }
  }
}

}  // namespace

int launch_anyblock(const GemmArgs& g, int64_t block_n, int64_t block_k, hipStream_t stream) {
  if (block_n < 1 || block_k < 1 || block_n > 0x7FFFFFFF || block_k > 0x7FFFFFFF)
    FG_FAIL(FG_ERR_INVALID_ARG, "block fp8 gemm: scale block %lld x %lld", (long long)block_n, (long long)block_k);
  AnyBlockArgs a;
  a.g = g;
  a.block_n = (int)block_n;
  a.block_k = (int)block_k;
  const bool mfma_ok = block_k % 32 == 0 && block_n % 16 == 0 && g.K % 16 == 0 && g.ldx % 16 == 0 && g.ldw % 16 == 0 &&
                       (uintptr_t)g.X % 16 == 0 && (uintptr_t)g.W % 16 == 0 && ceil_div((int64_t)g.M, (int64_t)kSubTile) <= 65535;
  if (mfma_ok) {
    FG_LAUNCH(block_fp8_gemm_subblock_kernel, dim3((uint32_t)ceil_div((int64_t)g.N, (int64_t)kSubTile), (uint32_t)ceil_div((int64_t)g.M, (int64_t)kSubTile)),
              dim3(kSubThreads), 0, stream, a);
    FG_CHECK_LAUNCH("block_fp8_gemm_subblock_kernel");
    return FG_OK;
  }
  const int64_t tiles_n = ceil_div((int64_t)g.N, (int64_t)kAnyTile), tiles_m = ceil_div((int64_t)g.M, (int64_t)kAnyTile);
  if (tiles_m > 65535) FG_FAIL(FG_ERR_UNSUPPORTED, "block fp8 gemm with %lld x %lld scale blocks: more than %d rows", (long long)block_n,
                               (long long)block_k, 65535 * kAnyTile);
  FG_LAUNCH(block_fp8_gemm_anyblock_kernel, dim3((uint32_t)tiles_n, (uint32_t)tiles_m), dim3(256), 0, stream, a);
  FG_CHECK_LAUNCH("block_fp8_gemm_anyblock_kernel");
  return FG_OK;
}

}  // namespace fg
