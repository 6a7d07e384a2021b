// aten::_scaled_mm for operands that are not quantized (bf16, fp16, fp32) on gfx950:
//     C[m, n] = cast( (sum_k A[m, k] * B[n, k]) * a_scale[m or 0] * b_scale[n or 0] + bias[n] )
// with the sum, the scales and the bias in fp32 and one rounding at the end, which is what the reference's generic
// kernel computes (src/flag_gems/ops/scaled_mm.py:77-133: tl.dot with an fp32 accumulator and allow_tf32 = False,
// acc * scale_a * scale_b, + bias, store).
//
// The quantized operand types have tuned kernels of their own; this one keeps the operator on the GPU for the
// other types.  A workgroup of four wavefronts computes a 128 x 128 tile of C, each wavefront a 64 x 64 quarter as
// 4 x 4 MFMA tiles (v_mfma_f32_16x16x32_bf16 / _f16, v_mfma_f32_16x16x4_f32).  Both operands are K-contiguous rows,
// and an MFMA operand is "row (lane % 16), eight consecutive k at 8 (lane / 16)": one 16-byte load per lane and
// tile straight from global memory, no LDS; the next K step's operands are loaded before the current step's
// MFMAs.  The two wavefronts that share a row or column panel meet in the L1/L2 caches.

#include "fg_common.h"
#include "fp8_gemm_common.h"

namespace fg {
namespace {

constexpr int kGenThreads = 256;
constexpr int kGenTile = 128;    // rows and columns of C per workgroup
constexpr int kGenWaveTile = 64; // per wavefront
constexpr int kGenFrags = kGenWaveTile / 16;

struct GenericArgs {
  const void* A;
  const void* B;
  int64_t lda, ldb, ldc;  // elements
  const float* a_scale;
  const float* b_scale;
  int a_per_row, b_per_col;
  const void* bias;
  int bias_dtype;
  void* C;
  int c_dtype;
  int M, N, K;
  int tiles_n;
};

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

template <int DT> struct GenElem;
template <> struct GenElem<FG_BF16> {
  static constexpr int kBytes = 2, kStep = 32;  // K per 16-byte load round: 4 lane groups x 8 elements
  __device__ static v4f mma(u32x4 a, u32x4 b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct GenElem<FG_F16> {
  static constexpr int kBytes = 2, kStep = 32;
  __device__ static v4f mma(u32x4 a, u32x4 b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct GenElem<FG_F32> {
  static constexpr int kBytes = 4, kStep = 16;  // 4 lane groups x 4 elements; element j of every lane feeds MFMA j
  __device__ static v4f mma(u32x4 a, u32x4 b, v4f c) {
#pragma unroll
    for (int j = 0; j < 4; ++j) c = __builtin_amdgcn_mfma_f32_16x16x4f32(bits_to_float(a[j]), bits_to_float(b[j]), c, 0, 0, 0);
    return c;
  }
};

__device__ __forceinline__ float load_scalar_as_float(const void* p, int64_t i, int dtype) {
  if (dtype == FG_F32) return reinterpret_cast<const float*>(p)[i];
  if (dtype == FG_F16) return (float)reinterpret_cast<const _Float16*>(p)[i];
  return bits_to_float((uint32_t)reinterpret_cast<const uint16_t*>(p)[i] << 16);
}

__device__ __forceinline__ void store_rounded(void* C, int64_t off, float v, int dtype) {
  if (dtype == FG_F32) {
    reinterpret_cast<float*>(C)[off] = v;
  } else if (dtype == FG_F16) {
    reinterpret_cast<_Float16*>(C)[off] = (_Float16)v;
  } else {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const uint32_t w = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{v, 0.0f}, bf16x2));
    reinterpret_cast<uint16_t*>(C)[off] = (uint16_t)(w & 0xFFFFu);
  }
}

template <int DT>
__global__ __launch_bounds__(kGenThreads) void scaled_gemm_generic_kernel(GenericArgs a) {
  using E = GenElem<DT>;
  constexpr int kPerLane = 16 / E::kBytes;  // elements of one 16-byte load
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile_m = blockIdx.x / a.tiles_n, tile_n = blockIdx.x - tile_m * a.tiles_n;
  const int m0 = tile_m * kGenTile + (wave >> 1) * kGenWaveTile;
  const int n0 = tile_n * kGenTile + (wave & 1) * kGenWaveTile;
  // a wavefront whose quarter lies outside C has nothing to do (there is no barrier in this kernel)
  if (m0 >= a.M || n0 >= a.N) return;

  const int r = lane & 15, kq = (lane >> 4) * kPerLane;
  // rows past the edge read the last valid row (their results are not stored)
  const char* ap[kGenFrags];
  const char* bp[kGenFrags];
#pragma unroll
  for (int f = 0; f < kGenFrags; ++f) {
    const int am = min(m0 + 16 * f + r, a.M - 1), bn = min(n0 + 16 * f + r, a.N - 1);
    ap[f] = reinterpret_cast<const char*>(a.A) + ((int64_t)am * a.lda + kq) * E::kBytes;
    bp[f] = reinterpret_cast<const char*>(a.B) + ((int64_t)bn * a.ldb + kq) * E::kBytes;
  }

  v4f acc[kGenFrags][kGenFrags];
#pragma unroll
  for (int i = 0; i < kGenFrags; ++i)
#pragma unroll
    for (int j = 0; j < kGenFrags; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  const u32x4 zero = {0u, 0u, 0u, 0u};
  u32x4 fa[kGenFrags], fb[kGenFrags], na[kGenFrags], nb[kGenFrags];
  // K is a multiple of the elements per load, so a lane's load lies wholly inside or wholly outside the row
  auto load_step = [&](int k, u32x4 (&xa)[kGenFrags], u32x4 (&xb)[kGenFrags]) {
    const bool inside = k + kq < a.K;
#pragma unroll
    for (int f = 0; f < kGenFrags; ++f) {
      xa[f] = inside ? *reinterpret_cast<const u32x4*>(ap[f] + (int64_t)k * E::kBytes) : zero;
      xb[f] = inside ? *reinterpret_cast<const u32x4*>(bp[f] + (int64_t)k * E::kBytes) : zero;
    }
  };

  load_step(0, fa, fb);
  for (int k = 0; k < a.K; k += E::kStep) {
    const bool more = k + E::kStep < a.K;  // uniform
    if (more) load_step(k + E::kStep, na, nb);
#pragma unroll
    for (int i = 0; i < kGenFrags; ++i)
#pragma unroll
      for (int j = 0; j < kGenFrags; ++j) acc[i][j] = E::mma(fa[i], fb[j], acc[i][j]);
    if (more) {
#pragma unroll
      for (int f = 0; f < kGenFrags; ++f) { fa[f] = na[f]; fb[f] = nb[f]; }
    }
  }

  // lane holds C[16 i + 4 (lane / 16) + e][16 j + lane % 16], e < 4
  const int crow = (lane >> 4) * 4, ccol = lane & 15;
#pragma unroll
  for (int j = 0; j < kGenFrags; ++j) {
    const int n = n0 + 16 * j + ccol;
    if (n >= a.N) continue;
    const float sb = a.b_scale[a.b_per_col ? n : 0];
    const float bias = a.bias ? load_scalar_as_float(a.bias, n, a.bias_dtype) : 0.0f;
#pragma unroll
    for (int i = 0; i < kGenFrags; ++i) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = m0 + 16 * i + crow + e;
        if (m >= a.M) continue;
        float v = (acc[i][j][e] * a.a_scale[a.a_per_row ? m : 0]) * sb;
        if (a.bias) v = v + bias;
        store_rounded(a.C, (int64_t)m * a.ldc + n, v, a.c_dtype);
      }
    }
  }
}

// The same tile for the 16-bit types with the operand panels staged through LDS, so that each is read from global
// memory once per workgroup instead of once per wavefront: per K step of 64 elements the 256 threads copy the
// 128 x 64 panels of A and B (16 KB each) into one of two LDS stages, 16 bytes per thread and access, rows 128 bytes
// apart with the 16-byte column XORed with (row & 7) so that the fragment reads (16 consecutive rows at one column)
// fall into different banks.  The global loads of step k + 1 are issued before the MFMAs of step k and written to the
// other stage after them; one barrier per step.  Measured on bf16 M = N = K = 4096: 495 us with the direct kernel, 202 us (680 TFLOP/s) with this one.
constexpr int kLdsStepElems = 64;                       // K per step (16-bit elements)
constexpr int kLdsRowBytes = kLdsStepElems * 2;         // 128
constexpr int kLdsPanelBytes = kGenTile * kLdsRowBytes; // 16 KB
constexpr int kLdsChunksPerThread = kGenTile * (kLdsRowBytes / 16) / kGenThreads;  // 4

__device__ __forceinline__ int lds_chunk_offset(int row, int chunk) { return row * kLdsRowBytes + ((chunk ^ (row & 7)) << 4); }

template <int DT>
__global__ __launch_bounds__(kGenThreads) void scaled_gemm_lds_kernel(GenericArgs a) {
  using E = GenElem<DT>;
  static_assert(E::kBytes == 2, "16-bit operands only");
  __shared__ __attribute__((aligned(16))) char lds[2][2][kLdsPanelBytes];  // [stage][A or B][panel]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tile_m = blockIdx.x / a.tiles_n, tile_n = blockIdx.x - tile_m * a.tiles_n;
  const int bm0 = tile_m * kGenTile, bn0 = tile_n * kGenTile;

  // copy duty of this thread: chunk column tid & 7 of rows (tid >> 3) + 32 i; rows past the edge read the last valid row
  const int cc = tid & 7, cr = tid >> 3;
  const char* ag[kLdsChunksPerThread];
  const char* bg[kLdsChunksPerThread];
  int lo[kLdsChunksPerThread];
#pragma unroll
  for (int i = 0; i < kLdsChunksPerThread; ++i) {
    const int row = cr + 32 * i;
    ag[i] = reinterpret_cast<const char*>(a.A) + ((int64_t)min(bm0 + row, a.M - 1) * a.lda + cc * 8) * 2;
    bg[i] = reinterpret_cast<const char*>(a.B) + ((int64_t)min(bn0 + row, a.N - 1) * a.ldb + cc * 8) * 2;
    lo[i] = lds_chunk_offset(row, cc);
  }
  const u32x4 zero = {0u, 0u, 0u, 0u};
  u32x4 ra[kLdsChunksPerThread], rb[kLdsChunksPerThread];
  // K is a multiple of 8: a chunk lies wholly inside or wholly outside the row
  auto fetch = [&](int k) {
    const bool inside = k + cc * 8 < a.K;
#pragma unroll
    for (int i = 0; i < kLdsChunksPerThread; ++i) {
      ra[i] = inside ? *reinterpret_cast<const u32x4*>(ag[i] + (int64_t)k * 2) : zero;
      rb[i] = inside ? *reinterpret_cast<const u32x4*>(bg[i] + (int64_t)k * 2) : zero;
    }
  };
  auto stash = [&](int stage) {
#pragma unroll
    for (int i = 0; i < kLdsChunksPerThread; ++i) {
      *reinterpret_cast<u32x4*>(&lds[stage][0][lo[i]]) = ra[i];
      *reinterpret_cast<u32x4*>(&lds[stage][1][lo[i]]) = rb[i];
    }
  };

  v4f acc[kGenFrags][kGenFrags];
#pragma unroll
  for (int i = 0; i < kGenFrags; ++i)
#pragma unroll
    for (int j = 0; j < kGenFrags; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  const int wm0 = (wave >> 1) * kGenWaveTile, wn0 = (wave & 1) * kGenWaveTile;  // inside the tile
  const int r = lane & 15, q = lane >> 4;

  fetch(0);
  stash(0);
  __syncthreads();
  int stage = 0;
  for (int k = 0; k < a.K; k += kLdsStepElems, stage ^= 1) {
    const bool more = k + kLdsStepElems < a.K;  // uniform over the workgroup
    if (more) fetch(k + kLdsStepElems);
#pragma unroll
    for (int h = 0; h < 2; ++h) {  // the two 32-element halves of the step
      u32x4 fa[kGenFrags], fb[kGenFrags];
#pragma unroll
      for (int f = 0; f < kGenFrags; ++f) {
        fa[f] = *reinterpret_cast<const u32x4*>(&lds[stage][0][lds_chunk_offset(wm0 + 16 * f + r, 4 * h + q)]);
        fb[f] = *reinterpret_cast<const u32x4*>(&lds[stage][1][lds_chunk_offset(wn0 + 16 * f + r, 4 * h + q)]);
      }
#pragma unroll
      for (int i = 0; i < kGenFrags; ++i)
#pragma unroll
        for (int j = 0; j < kGenFrags; ++j) acc[i][j] = E::mma(fa[i], fb[j], acc[i][j]);
    }
    if (more) stash(stage ^ 1);
    __syncthreads();  // the other stage is complete, and every read of this one is done before it is written again
  }

  const int m0 = bm0 + wm0, n0 = bn0 + wn0;
  const int crow = q * 4, ccol = r;
#pragma unroll
  for (int j = 0; j < kGenFrags; ++j) {
    const int n = n0 + 16 * j + ccol;
    if (n >= a.N) continue;
    const float sb = a.b_scale[a.b_per_col ? n : 0];
    const float bias = a.bias ? load_scalar_as_float(a.bias, n, a.bias_dtype) : 0.0f;
#pragma unroll
    for (int i = 0; i < kGenFrags; ++i) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = m0 + 16 * i + crow + e;
        if (m >= a.M) continue;
        float v = (acc[i][j][e] * a.a_scale[a.a_per_row ? m : 0]) * sb;
        if (a.bias) v = v + bias;
        store_rounded(a.C, (int64_t)m * a.ldc + n, v, a.c_dtype);
      }
    }
  }
}

// Up to 128 rows: 128 x 128 tiles would leave most compute units idle (M = 64, N = 4096: 32 tiles), and one K step per
// round trip to memory makes a lone tile a chain of load latencies.  Here a workgroup owns 16 columns of C for up to
// 64 rows; its eight wavefronts share K (wavefront w takes the runs of kSkinnySteps K steps numbered w, w + 8, ...),
// each keeps one run in flight beyond the one it multiplies, and their sums meet in LDS, added in wavefront order.
// B takes the first operand slot, so a lane's four results are four consecutive columns of one row.
// Measured, N = K = 4096: M = 64 bf16 62 -> 23 us, fp32 296 -> 50 us; M = 1 bf16 7.6 us (4.4 TB/s of weights), M = 16 10.4 us,
// M = 128 (two slices of 64 rows) 42 us.  With 64 rows a workgroup fetches four bytes of A for every byte of B, all from L2.
constexpr int kSkinnyWaves = 8;
constexpr int kSkinnySteps = 4;  // K steps per run

template <int DT, int FM>
__global__ __launch_bounds__(kSkinnyWaves * 64) void scaled_gemm_skinny_kernel(GenericArgs a) {
  using E = GenElem<DT>;
  constexpr int kPerLane = 16 / E::kBytes;
  constexpr int kRun = kSkinnySteps * E::kStep;  // elements of K per run
  __shared__ float sums[kSkinnyWaves][FM][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * 16, m0 = blockIdx.y * (16 * FM);
  const int r = lane & 15, kq = (lane >> 4) * kPerLane;
  // rows past the edge read the last valid row (their results are not stored)
  const char* const bp = reinterpret_cast<const char*>(a.B) + ((int64_t)min(n0 + r, a.N - 1) * a.ldb + kq) * E::kBytes;
  const char* ap[FM];
#pragma unroll
  for (int f = 0; f < FM; ++f)
    ap[f] = reinterpret_cast<const char*>(a.A) + ((int64_t)min(m0 + 16 * f + r, a.M - 1) * a.lda + kq) * E::kBytes;

  v4f acc[FM];
#pragma unroll
  for (int f = 0; f < FM; ++f) acc[f] = v4f{0.f, 0.f, 0.f, 0.f};

  const u32x4 zero = {0u, 0u, 0u, 0u};
  u32x4 cb[kSkinnySteps], ca[kSkinnySteps][FM], nb[kSkinnySteps], na[kSkinnySteps][FM];
  // K is a multiple of the elements per load, so a lane's load lies wholly inside or wholly outside the row
  auto load_run = [&](int run, u32x4 (&xb)[kSkinnySteps], u32x4 (&xa)[kSkinnySteps][FM]) {
#pragma unroll
    for (int u = 0; u < kSkinnySteps; ++u) {
      const int k = run * kRun + u * E::kStep;
      const bool inside = k + kq < a.K;
      xb[u] = inside ? *reinterpret_cast<const u32x4*>(bp + (int64_t)k * E::kBytes) : zero;
#pragma unroll
      for (int f = 0; f < FM; ++f) xa[u][f] = inside ? *reinterpret_cast<const u32x4*>(ap[f] + (int64_t)k * E::kBytes) : zero;
    }
  };

  const int runs = (a.K + kRun - 1) / kRun;
  if (wave < runs) load_run(wave, cb, ca);
  for (int run = wave; run < runs; run += kSkinnyWaves) {
    const bool more = run + kSkinnyWaves < runs;  // uniform over the wavefront
    if (more) load_run(run + kSkinnyWaves, nb, na);
#pragma unroll
    for (int u = 0; u < kSkinnySteps; ++u)
#pragma unroll
      for (int f = 0; f < FM; ++f) acc[f] = E::mma(cb[u], ca[u][f], acc[f]);
    if (more) {
#pragma unroll
      for (int u = 0; u < kSkinnySteps; ++u) {
        cb[u] = nb[u];
#pragma unroll
        for (int f = 0; f < FM; ++f) ca[u][f] = na[u][f];
      }
    }
  }

  // lane holds C[m0 + 16 f + lane % 16][n0 + 4 (lane / 16) + e], e < 4
#pragma unroll
  for (int f = 0; f < FM; ++f)
#pragma unroll
    for (int e = 0; e < 4; ++e) sums[wave][f][e][lane] = acc[f][e];
  __syncthreads();
  for (int o = threadIdx.x; o < FM * 256; o += kSkinnyWaves * 64) {
    const int f = o >> 8, ml = (o >> 4) & 15, nl = o & 15;
    const int m = m0 + 16 * f + ml, n = n0 + nl;
    if (m >= a.M || n >= a.N) continue;
    const int src = (nl >> 2) * 16 + ml, e = nl & 3;
    float v = sums[0][f][e][src];
#pragma unroll
    for (int w = 1; w < kSkinnyWaves; ++w) v = v + sums[w][f][e][src];
    v = (v * a.a_scale[a.a_per_row ? m : 0]) * a.b_scale[a.b_per_col ? n : 0];
    if (a.bias) v = v + load_scalar_as_float(a.bias, n, a.bias_dtype);
    store_rounded(a.C, (int64_t)m * a.ldc + n, v, a.c_dtype);
  }
}

template <int DT>
void launch_skinny(const GenericArgs& g, hipStream_t stream) {
  const int slices = (g.M + 63) / 64;                    // of up to 64 rows each
  const int fm = ((g.M + slices - 1) / slices + 15) / 16;
  const dim3 grid((uint32_t)((g.N + 15) / 16), (uint32_t)((g.M + 16 * fm - 1) / (16 * fm))), block(kSkinnyWaves * 64);
  switch (fm) {
    case 1: FG_LAUNCH((scaled_gemm_skinny_kernel<DT, 1>), grid, block, 0, stream, g); break;
    case 2: FG_LAUNCH((scaled_gemm_skinny_kernel<DT, 2>), grid, block, 0, stream, g); break;
    case 3: FG_LAUNCH((scaled_gemm_skinny_kernel<DT, 3>), grid, block, 0, stream, g); break;
    default: FG_LAUNCH((scaled_gemm_skinny_kernel<DT, 4>), grid, block, 0, stream, g); break;
  }
}

}  // namespace
}  // namespace fg

extern "C" int fg_scaled_gemm(const void* A, int64_t lda, const void* B, int64_t ldb, int ab_dtype,
                              const float* a_scale, int a_scale_per_row,
                              const float* b_scale, int b_scale_per_col,
                              const void* bias, int bias_dtype,
                              void* C, int64_t ldc, int c_dtype,
                              int64_t M, int64_t N, int64_t K, void* stream) {
  using namespace fg;
  const char* me = "fg_scaled_gemm";
  if (M < 0 || N < 0 || K < 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: negative size", me);
  if (M == 0 || N == 0) return FG_OK;
  if (!A || !B || !C || !a_scale || !b_scale) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null pointer", me);
  if (ab_dtype != FG_BF16 && ab_dtype != FG_F16 && ab_dtype != FG_F32) FG_FAIL(FG_ERR_INVALID_ARG, "%s: operand dtype %d", me, ab_dtype);
  if (c_dtype != FG_BF16 && c_dtype != FG_F16 && c_dtype != FG_F32) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: output dtype %d", me, c_dtype);
  if (bias && bias_dtype != FG_BF16 && bias_dtype != FG_F16 && bias_dtype != FG_F32)
    FG_FAIL(FG_ERR_INVALID_ARG, "%s: bias dtype %d", me, bias_dtype);
  if (lda < K || ldb < K || ldc < N) FG_FAIL(FG_ERR_INVALID_ARG, "%s: row stride smaller than the row", me);
  if (M > 0x3FFFFFFF || N > 0x3FFFFFFF || K > 0x3FFFFFFF) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: dimension above 2^30", me);
  const int64_t esz = ab_dtype == FG_F32 ? 4 : 2, per_load = 16 / esz;
  if (K % per_load != 0 || (uintptr_t)A % 16 != 0 || (uintptr_t)B % 16 != 0 || (lda * esz) % 16 != 0 || (ldb * esz) % 16 != 0)
    FG_FAIL(FG_ERR_UNSUPPORTED, "%s: K must be a multiple of %lld and operand rows 16-byte aligned", me, (long long)per_load);
  const int64_t tiles_m = ceil_div(M, kGenTile), tiles_n = ceil_div(N, kGenTile);
  if (tiles_m * tiles_n > 0x7FFFFFFF) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: too many tiles", me);

  // 16-bit operands and results, more than 128 rows, whole 128-byte K-blocks: the persistent kernel of the fp8 GEMMs,
  // which takes operand rows as bytes
  // (M = N = K = 4096, bf16: 202 -> 126 us, 1.09 PFLOP/s; 8192^3: 1314 -> 773 us, 1.42 PFLOP/s).  Without a workspace
  // its tiles are never shared along K, so it needs 256 x 256 tiles for most of the compute units: M = 1024, N = 4096
  // (64 tiles) takes 88 us there against 70 us below.
  if (ab_dtype != FG_F32 && M > 128 && K % 64 == 0 && K > 0 && lda * 2 < (1 << 23) && ldb * 2 < (1 << 23) &&
      ceil_div(M, 256) * ceil_div(N, 256) * 5 >= (int64_t)cu_count() * 3) {
    GemmArgs p = {};
    p.X = reinterpret_cast<const uint8_t*>(A); p.W = reinterpret_cast<const uint8_t*>(B); p.C = C;
    p.xs = a_scale; p.ws = b_scale; p.bias = bias;
    p.ldx = lda * 2; p.ldw = ldb * 2; p.ldc = ldc;
    p.M = (int)M; p.N = (int)N; p.K = (int)(K * 2); p.KB = (int)(K / 64);
    p.c_dtype = c_dtype; p.bias_dtype = bias_dtype;
    p.xs_per_row = a_scale_per_row; p.ws_per_col = b_scale_per_col;
    const int mode = ab_dtype == FG_BF16 ? kModeRowColBF16 : kModeRowColF16;
    if (pingpong_takes(p, mode, nullptr, 0)) return launch_pingpong(p, mode, nullptr, 0, (hipStream_t)stream);
  }

  GenericArgs g;
  g.A = A; g.B = B; g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.a_scale = a_scale; g.b_scale = b_scale;
  g.a_per_row = a_scale_per_row != 0; g.b_per_col = b_scale_per_col != 0;
  g.bias = bias; g.bias_dtype = bias_dtype;
  g.C = C; g.c_dtype = c_dtype;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  g.tiles_n = (int)tiles_n;
  // Up to 128 rows: workgroups of 16 columns while that is the faster way.  Their time grows with N (every workgroup
  // fetches the rows of A again), the 128 x 128 tiles' time only with the rounds of tiles over the compute units.
  // Timed on both at K = 4096, us: bf16 M = 64: N = 8192 43 against 63, N = 16384 83 against 65; M = 128: N = 4096 44 against
  // 64, N = 8192 84 against 64; fp32 M = 64: N = 16384 194 against 299, N = 28672 352 against 301; both scale with K.
  // (With at most 32 rows of 16-bit operands the tiles load straight from global memory, 74-95 us: never faster.)
  bool skinny = M <= 128 && ceil_div(N, 16) <= 0x7FFFFFFF;
  if (skinny && (ab_dtype == FG_F32 || M > 32)) {
    const int64_t slices = ceil_div(M, 64), fm = ceil_div(ceil_div(M, slices), 16);
    const double k4 = (double)K / 4096.0, units = (double)ceil_div(N, 16) * (double)slices * (double)(fm + 1);
    const double rounds = (double)ceil_div(tiles_m * tiles_n, (int64_t)cu_count());
    const double t_skinny = 3.0 + (ab_dtype == FG_F32 ? 0.037 : 0.0155) * units * k4;
    const double t_tiles = (ab_dtype == FG_F32 ? 5.0 + 290.0 * k4 : 10.0 + 52.0 * k4) * rounds;
    skinny = t_skinny < t_tiles;
  }
  if (skinny) {
    if (ab_dtype == FG_BF16) launch_skinny<FG_BF16>(g, (hipStream_t)stream);
    else if (ab_dtype == FG_F16) launch_skinny<FG_F16>(g, (hipStream_t)stream);
    else launch_skinny<FG_F32>(g, (hipStream_t)stream);
    FG_CHECK_LAUNCH("scaled_gemm_skinny_kernel");
    return FG_OK;
  }
  const dim3 grid((uint32_t)(tiles_m * tiles_n)), block(kGenThreads);
  // 16-bit operands with enough rows to fill tiles go through LDS; fp32 and short problems load straight into registers
  const bool staged = ab_dtype != FG_F32 && M > 32 && K >= kLdsStepElems;
  if (staged && ab_dtype == FG_BF16) FG_LAUNCH(scaled_gemm_lds_kernel<FG_BF16>, grid, block, 0, (hipStream_t)stream, g);
  else if (staged) FG_LAUNCH(scaled_gemm_lds_kernel<FG_F16>, grid, block, 0, (hipStream_t)stream, g);
  else if (ab_dtype == FG_BF16) FG_LAUNCH(scaled_gemm_generic_kernel<FG_BF16>, grid, block, 0, (hipStream_t)stream, g);
  else if (ab_dtype == FG_F16) FG_LAUNCH(scaled_gemm_generic_kernel<FG_F16>, grid, block, 0, (hipStream_t)stream, g);
  else FG_LAUNCH(scaled_gemm_generic_kernel<FG_F32>, grid, block, 0, (hipStream_t)stream, g);
  FG_CHECK_LAUNCH("scaled_gemm_generic_kernel");
  return FG_OK;
}
