// RMSNorm fused into the per-token-group FP8 quantizer for gfx950: the normalised activation goes from registers
// straight into the quantizer, so the 16-bit tensor between the norm and the quantized linear layer is neither
// written nor read again.
//
// One workgroup of 256 threads owns a row at a time (and walks rows with the grid's stride).  Thread t holds the
// 8-element chunks t, t + 256, ... of the row in registers, so 16 (or 8) adjacent lanes hold one quantization
// group, as in the plain quantizer.  The sum of squares is accumulated per thread in chunk order, folded across the
// 64 lanes with a butterfly and across the four wavefronts through LDS in wavefront order; every step is an
// individually rounded fp32 operation, so the result does not depend on how the compiler contracts it.
//
// Arithmetic follows the reference's two operators:
//   without residual (src/flag_gems/ops/rms_norm.py:54-66): var = sum(x^2) / N, rrms = 1 / sqrt(var + eps),
//     y = T(T(x * rrms) * w), T = rounding to x's type;
//   with residual (src/flag_gems/fused/fused_add_rms_norm.py:92-118, the looped form): t = x + residual in fp32,
//     residual <- T(t), var = sum(t^2) / N over the unrounded t, y = T(T(t) * rrms * w).
// The reference leaves the order of the sum to its compiler; the order above is this library's.

#include "fp8_quant_device.h"

// every fp32 operation of this file is rounded on its own: the sum of squares and the normalisation must not depend
// on which multiplies the compiler would fuse into the following add
#pragma clang fp contract(off)

namespace fg {
namespace {

constexpr int kNormThreads = 256;
constexpr int kNormWaves = kNormThreads / 64;
constexpr int kNormMaxChunks = 8;  // chunks per thread: rows of up to 8 * 256 * 8 = 16384 elements

struct NormQuantArgs {
  QuantArgs q;             // q.x = input; q.q / q.s may be null (normalise only)
  void* residual;          // null, or [rows, cols] added to x and overwritten with the sum
  const void* weight;      // [cols], x's type
  void* y;                 // null, or [rows, cols] normalised output in x's type (may alias x)
  int64_t residual_row_stride, y_row_stride;
  uint32_t rows, chunks_per_row, lanes_per_group;
  float eps, n_as_float;
};

// max over `lanes` adjacent lanes (a power of two up to 64), every lane ends with the group's value
__device__ __forceinline__ uint32_t group_max_lanes(uint32_t v, uint32_t lanes) {
  if (lanes >= 2) v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true));
  if (lanes >= 4) v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true));
  if (lanes >= 8) v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x141, 0xF, 0xF, true));
  if (lanes >= 16) v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x140, 0xF, 0xF, true));
  if (lanes >= 32) v = max(v, (uint32_t)__shfl_xor((int)v, 16, 64));
  if (lanes >= 64) v = max(v, (uint32_t)__shfl_xor((int)v, 32, 64));
  return v;
}

// value + value of the lane whose index differs in bit `mask`, for every lane
__device__ __forceinline__ float butterfly_add(float v, int mask) { return v + __shfl_xor(v, mask, 64); }

template <int XDT, int WORDS>
__device__ __forceinline__ void load_chunk(const typename Elem<XDT>::raw* p, uint32_t (&w)[WORDS]) {
#pragma unroll
  for (int k = 0; k < WORDS / 4; ++k) {
    const u32x4 v = reinterpret_cast<const u32x4*>(p)[k];
    w[4 * k] = v.x; w[4 * k + 1] = v.y; w[4 * k + 2] = v.z; w[4 * k + 3] = v.w;
  }
}
template <int XDT, int WORDS>
__device__ __forceinline__ void store_chunk(typename Elem<XDT>::raw* p, const uint32_t (&w)[WORDS]) {
#pragma unroll
  for (int k = 0; k < WORDS / 4; ++k) {
    const u32x4 v = {w[4 * k], w[4 * k + 1], w[4 * k + 2], w[4 * k + 3]};
    reinterpret_cast<u32x4*>(p)[k] = v;
  }
}
// eight fp32 values -> the raw words of x's type (rounded to nearest even)
template <int XDT, int WORDS>
__device__ __forceinline__ void narrow_chunk(const float (&v)[8], uint32_t (&w)[WORDS]) {
  if constexpr (WORDS == 4) {
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = Elem<XDT>::narrow2(v[2 * i], v[2 * i + 1]);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = float_to_bits(v[i]);
  }
}

// Measured on bf16 [4096, 7168]: 25 us for the norm alone (4.7 TB/s), 36 us with the quantizer (the quantizer alone:
// 18 us): with both in one kernel the vector ALU is the limit, not memory.  A variant with as many workgroups as stay
// resident, each loading its next row (raw words) before working on the current one, was measured and not kept: the
// norm alone went to 22.5 us, the fused call stayed at 37 us, and rows of 16384 elements got slower (150 us against
// 101) because the second row in registers left one wavefront per SIMD.
// QUANT: 0 = the norm alone, 1 = with the quantizer and its rules taken from the arguments, 2 = with the quantizer
// under the rules of per_token_group_quant_fp8's defaults (scale = amax * (1 / max), true division, no power-of-two
// rounding, e4m3), which lets the compiler drop every rule switch from the loop.
// LPG: lanes per quantization group when known at compile time (16 = groups of 128 elements), 0 = from the arguments:
// the group maximum is then four DPP instructions instead of a chain of six tests.
// A wavefront whose 64 chunks of a pass all lie past the row's end (rows of 7168 elements: the last pass of
// wavefronts 2 and 3) skips the pass; its zeros would not have changed any sum.
template <int XDT, int CHUNKS, int QUANT, int LPG = 0>
__global__ __launch_bounds__(kNormThreads) void rms_norm_quant_kernel(NormQuantArgs a) {
  if (QUANT == 2) {
    a.q.scale_rule = FG_SCALE_MUL_INV;
    a.q.quotient_rule = FG_QUOT_DIV;
    a.q.pow2_rule = FG_POW2_NONE;
    a.q.e5m2 = 0;
  }
  using E = Elem<XDT>;
  using Raw = typename E::raw;
  constexpr int kWords = sizeof(Raw) * 8 / 4;
  __shared__ float wave_sums[2][kNormWaves];

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t wave_first = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid & ~63u));  // chunk of lane 0 in the first pass over the row
  const bool add_residual = a.residual != nullptr;
  constexpr bool quantize = QUANT != 0;
  const Raw* wp = reinterpret_cast<const Raw*>(a.weight);
  uint32_t parity = 0;

  for (uint32_t row = blockIdx.x; row < a.rows; row += gridDim.x, parity ^= 1u) {
    const Raw* xp = reinterpret_cast<const Raw*>(a.q.x) + (int64_t)row * a.q.x_row_stride;
    Raw* rp = add_residual ? reinterpret_cast<Raw*>(a.residual) + (int64_t)row * a.residual_row_stride : nullptr;

    // the row (plus residual) in fp32, eight values per chunk; dead chunks hold zeros
    float v[CHUNKS][8];
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const uint32_t c = tid + (uint32_t)i * kNormThreads;
      const bool live = c < a.chunks_per_row;
      if (wave_first + (uint32_t)i * kNormThreads >= a.chunks_per_row) {  // uniform: this wavefront holds nothing of this pass
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = 0.0f;
        continue;
      }
      uint32_t rw[kWords];
      if (live) {
        uint32_t w[kWords];
        load_chunk<XDT, kWords>(xp + (size_t)c * 8, w);
        widen_chunk<XDT, kWords>(w, v[i]);
        if (add_residual) {
          float rv[8];
          load_chunk<XDT, kWords>(rp + (size_t)c * 8, rw);
          widen_chunk<XDT, kWords>(rw, rv);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[i][e] = v[i][e] + rv[e];
          narrow_chunk<XDT, kWords>(v[i], rw);
          store_chunk<XDT, kWords>(rp + (size_t)c * 8, rw);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = 0.0f;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) acc = acc + v[i][e] * v[i][e];  // two roundings (contraction is off in this file)
      // the reference's second pass reads the sum back as stored: rounded to the tensor's type
      if (live && add_residual) widen_chunk<XDT, kWords>(rw, v[i]);
    }

    // sum of squares of the row: lanes (butterfly, distances 1, 2, 4, 8, 16, 32), then wavefronts 0..3 in order
    acc = butterfly_add(acc, 1);
    acc = butterfly_add(acc, 2);
    acc = butterfly_add(acc, 4);
    acc = butterfly_add(acc, 8);
    acc = butterfly_add(acc, 16);
    acc = butterfly_add(acc, 32);
    if (lane == 0) wave_sums[parity][wave] = acc;
    __syncthreads();  // the other slot is written next: this barrier also orders its last reads before that
    float total = wave_sums[parity][0];
#pragma unroll
    for (int k = 1; k < kNormWaves; ++k) total = total + wave_sums[parity][k];
    const float var = total / a.n_as_float;                 // IEEE division and square root: correctly rounded
    const float rrms = 1.0f / __builtin_sqrtf(var + a.eps);

#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const uint32_t c = tid + (uint32_t)i * kNormThreads;
      const bool live = c < a.chunks_per_row;
      if (wave_first + (uint32_t)i * kNormThreads >= a.chunks_per_row) continue;
      uint32_t ww[kWords];
      float wv[8];
      if (live) load_chunk<XDT, kWords>(wp + (size_t)c * 8, ww);
      else {
#pragma unroll
        for (int k = 0; k < kWords; ++k) ww[k] = 0u;
      }
      widen_chunk<XDT, kWords>(ww, wv);
      uint32_t yw[kWords];
      if (add_residual) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = (v[i][e] * rrms) * wv[e];
        narrow_chunk<XDT, kWords>(v[i], yw);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = v[i][e] * rrms;
        narrow_chunk<XDT, kWords>(v[i], yw);
        float xn[8];
        widen_chunk<XDT, kWords>(yw, xn);
#pragma unroll
        for (int e = 0; e < 8; ++e) xn[e] = xn[e] * wv[e];
        narrow_chunk<XDT, kWords>(xn, yw);
      }
      if (live && a.y) store_chunk<XDT, kWords>(reinterpret_cast<Raw*>(a.y) + (int64_t)row * a.y_row_stride + (size_t)c * 8, yw);
      if (quantize) {  // uniform over the workgroup
        float yv[8];
        const uint32_t own = widen_chunk<XDT, kWords>(yw, yv);
        const uint32_t m = LPG != 0 ? group_max_u32<LPG>(own) : group_max_lanes(own, a.lanes_per_group);
        uint32_t w0, w1;
        const float s = quantize_chunk<XDT>(yv, m, a.q, w0, w1);
        if (live) {
          const u32x2 out = {w0, w1};
          *reinterpret_cast<u32x2*>(a.q.q + (int64_t)row * a.q.q_row_stride + (size_t)c * 8) = out;
          const uint32_t lpg = LPG != 0 ? (uint32_t)LPG : a.lanes_per_group;
          if (c % lpg == 0)
            a.q.s[(int64_t)row * a.q.s_row_stride + (int64_t)(c / lpg) * a.q.s_col_stride] = s;
        }
      }
    }
  }
}

template <int XDT>
int launch_norm(const NormQuantArgs& a, int cus, hipStream_t stream) {
  const uint32_t per_thread = (a.chunks_per_row + kNormThreads - 1) / kNormThreads;
  // enough workgroups to hold every compute unit's wave slots a few times over; beyond that, rows are walked
  const uint32_t grid = a.rows < (uint32_t)cus * 16u ? a.rows : (uint32_t)cus * 16u;
  const dim3 g(grid), b(kNormThreads);
  const int quant = a.q.q == nullptr ? 0
                    : (a.q.scale_rule == FG_SCALE_MUL_INV && a.q.quotient_rule == FG_QUOT_DIV && a.q.pow2_rule == FG_POW2_NONE && !a.q.e5m2) ? 2 : 1;
#define FG_NORM_LAUNCH(C)                                                                                            \
  do {                                                                                                               \
    if (quant == 0) FG_LAUNCH((rms_norm_quant_kernel<XDT, C, 0>), g, b, 0, stream, a);                      \
    else if (quant == 1) FG_LAUNCH((rms_norm_quant_kernel<XDT, C, 1>), g, b, 0, stream, a);                 \
    else if (a.lanes_per_group == 16) FG_LAUNCH((rms_norm_quant_kernel<XDT, C, 2, 16>), g, b, 0, stream, a); \
    else FG_LAUNCH((rms_norm_quant_kernel<XDT, C, 2>), g, b, 0, stream, a);                                 \
  } while (0)
  if (per_thread <= 1) FG_NORM_LAUNCH(1);
  else if (per_thread <= 2) FG_NORM_LAUNCH(2);
  else if (per_thread <= 4) FG_NORM_LAUNCH(4);
  else FG_NORM_LAUNCH(8);
#undef FG_NORM_LAUNCH
  FG_CHECK_LAUNCH("rms_norm_quant_kernel");
  return FG_OK;
}

}  // namespace
}  // namespace fg

extern "C" int fg_rms_norm_group_quant_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride,
                                           void* residual, int64_t residual_row_stride, const void* weight, float eps,
                                           void* y, int64_t y_row_stride,
                                           void* q, int q_dtype, int64_t q_row_stride,
                                           float* s, int64_t s_row_stride, int64_t s_col_stride,
                                           int64_t group_size, float amax_floor, float fp8_min, float fp8_max,
                                           float inv_fp8_max, int scale_rule, int quotient_rule, int pow2_rule,
                                           void* stream) {
  using namespace fg;
  const char* me = "fg_rms_norm_group_quant_fp8";
  if (rows < 0 || cols < 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: negative size", me);
  if (rows == 0 || cols == 0) return FG_OK;
  if (!x || !weight) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null input or weight", me);
  if ((q == nullptr) != (s == nullptr)) FG_FAIL(FG_ERR_INVALID_ARG, "%s: codes and scales come together", me);
  if (!q && !y) FG_FAIL(FG_ERR_INVALID_ARG, "%s: no output requested", me);
  if (x_dtype != FG_BF16 && x_dtype != FG_F16 && x_dtype != FG_F32) FG_FAIL(FG_ERR_INVALID_ARG, "%s: x_dtype %d", me, x_dtype);
  const int64_t esz = (x_dtype == FG_F32) ? 4 : 2;
  if (x_row_stride < cols || (residual && residual_row_stride < cols) || (y && y_row_stride < cols) ||
      (q && q_row_stride < cols))
    FG_FAIL(FG_ERR_INVALID_ARG, "%s: row stride smaller than cols", me);
  if (rows > 0x7FFFFFFF) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: more than 2^31 rows", me);
  if (cols % 8 != 0 || cols > (int64_t)kNormMaxChunks * kNormThreads * 8)
    FG_FAIL(FG_ERR_UNSUPPORTED, "%s: cols must be a multiple of 8 and at most %d, got %lld", me,
            kNormMaxChunks * kNormThreads * 8, (long long)cols);
  auto aligned = [&](const void* p, int64_t stride, int64_t bytes_per) {
    return (uintptr_t)p % 16 == 0 && (stride * bytes_per) % 16 == 0;
  };
  if (!aligned(x, x_row_stride, esz) || (uintptr_t)weight % 16 != 0 || (residual && !aligned(residual, residual_row_stride, esz)) ||
      (y && !aligned(y, y_row_stride, esz)))
    FG_FAIL(FG_ERR_UNSUPPORTED, "%s: rows must be 16-byte aligned", me);

  NormQuantArgs a;
  a.q.x = x;
  a.q.q = (uint8_t*)q;
  a.q.s = s;
  a.q.x_row_stride = x_row_stride;
  a.q.q_row_stride = q_row_stride;
  a.q.s_row_stride = s_row_stride;
  a.q.s_col_stride = s_col_stride;
  a.q.groups_per_row = 0;
  a.q.total_groups = 0;
  a.q.group_size = (uint32_t)group_size;
  a.q.floor = amax_floor;
  a.q.lo = fp8_min;
  a.q.hi = fp8_max;
  a.q.inv_max = inv_fp8_max;
  a.q.scale_rule = scale_rule;
  a.q.quotient_rule = quotient_rule;
  a.q.pow2_rule = pow2_rule;
  a.q.e5m2 = (q_dtype == FG_FP8_E5M2);
  a.q.up_offset = 0;
  a.q.inv_groups_per_row = 0.0f;
  a.lanes_per_group = 1;
  if (q) {
    if (q_dtype != FG_FP8_E4M3FN && q_dtype != FG_FP8_E5M2) FG_FAIL(FG_ERR_INVALID_ARG, "%s: q_dtype %d", me, q_dtype);
    if (scale_rule < 0 || scale_rule > 1 || quotient_rule < 0 || quotient_rule > 1 || pow2_rule < 0 || pow2_rule > 3)
      FG_FAIL(FG_ERR_INVALID_ARG, "%s: bad rule selector", me);
    if (group_size <= 0 || cols % group_size != 0)
      FG_FAIL(FG_ERR_INVALID_ARG, "%s: cols %lld not divisible by group_size %lld", me, (long long)cols, (long long)group_size);
    const int64_t lanes = group_size / 8;
    if (group_size % 8 != 0 || lanes > 64 || (lanes & (lanes - 1)) != 0)
      FG_FAIL(FG_ERR_UNSUPPORTED, "%s: group size must be 8, 16, 32, ... or 512", me);
    if ((uintptr_t)q % 8 != 0 || q_row_stride % 8 != 0) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: code rows must be 8-byte aligned", me);
    a.lanes_per_group = (uint32_t)lanes;
    a.q.groups_per_row = (uint32_t)(cols / group_size);
  }
  a.residual = residual;
  a.weight = weight;
  a.y = y;
  a.residual_row_stride = residual_row_stride;
  a.y_row_stride = y_row_stride;
  a.rows = (uint32_t)rows;
  a.chunks_per_row = (uint32_t)(cols / 8);
  a.eps = eps;
  a.n_as_float = (float)cols;

  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  if (x_dtype == FG_BF16) return launch_norm<FG_BF16>(a, cus, (hipStream_t)stream);
  if (x_dtype == FG_F16) return launch_norm<FG_F16>(a, cus, (hipStream_t)stream);
  return launch_norm<FG_F32>(a, cus, (hipStream_t)stream);
}
