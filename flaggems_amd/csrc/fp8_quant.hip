// Per-token-group FP8 quantizer for gfx950.
//
// One group of G consecutive elements is owned by G/8 adjacent lanes of a wavefront; every lane
// loads 8 elements with one (bf16/f16) or two (f32) 16-byte loads, the group's absolute maximum is
// reduced across those lanes with DPP / cross-lane moves, the scale is derived redundantly in every
// lane, and each lane writes its 8 codes with one 8-byte store.  The kernel is pure streaming:
// 2 (or 4) bytes read and 1 byte written per element plus 4 bytes of scale per group.
//
// Arithmetic is IEEE fp32 throughout (correctly rounded multiply, reciprocal and division) so the
// codes and scales are bit-identical to the torch reference implementations:
//   tests/test_act_quant.py:48-98 and tests/test_per_token_group_quant_fp8.py:23-48 of the reference.

#include "fp8_quant_device.h"

namespace fg {
namespace {


constexpr int kQuantThreads = 256;
// Independent 8-element chunks per thread (UNROLL of the vector kernel), loaded before any is converted.  Measured,
// bf16, group 128: two chunks are fastest on large inputs ([4096, 7168]: 18.2 us with four, 16.9 with two,
// 17.3 with one; [8192, 14336]: 67.6 / 66.4 / 73.9); inputs with fewer chunks than the GPU has lanes run one
// ([64, 7168]: 4.2 / 3.1 / 2.6 us).
constexpr int kQuantUnrollLarge = 2;
constexpr uint64_t kQuantSmallChunks = 512ull * 1024;  // up to this many chunks: one per thread

// Vector kernel: group_size == 8 * LPG, rows 16-byte aligned.
// SILU: the value quantized is silu(x[row, c]) * x[row, c + up_offset], rounded to x's type first (what a separate
// activation kernel would have stored), and x is never re-read.
// RULES: 0 = scale, quotient and rounding rules from the arguments; 1 = act_quant's defaults (amax * (1 / max),
// x * (1 / s), no power-of-two rounding, e4m3); 2 = per_token_group_quant_fp8's (the same with true division): the
// compiler then drops every rule switch from the loop.
template <int XDT, int LPG, int kQuantUnroll, bool SILU = false, int RULES = 0>
__global__ __launch_bounds__(kQuantThreads) void group_quant_vec_kernel(QuantArgs a) {
  if (RULES != 0) {
    a.scale_rule = FG_SCALE_MUL_INV;
    a.quotient_rule = RULES == 1 ? FG_QUOT_RECIP_MUL : FG_QUOT_DIV;
    a.pow2_rule = FG_POW2_NONE;
    a.e5m2 = 0;
  }
  using E = Elem<XDT>;
  constexpr int kWords = sizeof(typename E::raw) * 8 / 4;  // 32-bit words per lane: 4 or 8
  const uint32_t total_chunks = a.total_groups * (uint32_t)LPG;  // host guarantees no overflow
  const uint32_t stride = gridDim.x * kQuantThreads;
  const uint32_t first = blockIdx.x * kQuantThreads + threadIdx.x;

  uint32_t w[kQuantUnroll][kWords];
  uint32_t gid[kQuantUnroll], row[kQuantUnroll], gcol[kQuantUnroll];
  bool live[kQuantUnroll];

#pragma unroll
  for (int u = 0; u < kQuantUnroll; ++u) {
    uint32_t c = first + (uint32_t)u * stride;
    live[u] = c < total_chunks && c >= first;  // second test: wrap-around guard
    uint32_t cc = live[u] ? c : 0u;
    gid[u] = cc / LPG;
    uint32_t lig = cc % LPG;
    row[u] = divide_below_2_24(gid[u], a.groups_per_row, a.inv_groups_per_row, gcol[u]);
    const typename E::raw* p = reinterpret_cast<const typename E::raw*>(a.x) +
                               (int64_t)row[u] * a.x_row_stride + (int64_t)gcol[u] * (LPG * 8) + lig * 8;
    const u32x4* p4 = reinterpret_cast<const u32x4*>(p);
    if (live[u]) {
      u32x4 v = p4[0];
      w[u][0] = v.x; w[u][1] = v.y; w[u][2] = v.z; w[u][3] = v.w;
      if constexpr (kWords == 8) {
        u32x4 v2 = p4[1];
        w[u][4] = v2.x; w[u][5] = v2.y; w[u][6] = v2.z; w[u][7] = v2.w;
      }
      if constexpr (SILU) {
        const u32x4* q4 = reinterpret_cast<const u32x4*>(p + a.up_offset);
        uint32_t up[kWords];
        u32x4 t = q4[0];
        up[0] = t.x; up[1] = t.y; up[2] = t.z; up[3] = t.w;
        if constexpr (kWords == 8) {
          u32x4 t2 = q4[1];
          up[4] = t2.x; up[5] = t2.y; up[6] = t2.z; up[7] = t2.w;
        }
        silu_mul_words<XDT, kWords>(w[u], up);
      }
    } else {
#pragma unroll
      for (int i = 0; i < kWords; ++i) w[u][i] = 0u;
    }
  }

#pragma unroll
  for (int u = 0; u < kQuantUnroll; ++u) {
    float xv[8];
    const uint32_t m = group_max_u32<LPG>(widen_chunk<XDT, kWords>(w[u], xv));
    uint32_t w0, w1;
    const float s = quantize_chunk<XDT>(xv, m, a, w0, w1);
    if (live[u]) {
      uint32_t c = first + (uint32_t)u * stride;
      uint32_t lig = c % LPG;
      uint8_t* qp = a.q + (int64_t)row[u] * a.q_row_stride + (int64_t)gcol[u] * (LPG * 8) + lig * 8;
      u32x2 out = {w0, w1};
      *reinterpret_cast<u32x2*>(qp) = out;
      if (lig == 0) a.s[(int64_t)row[u] * a.s_row_stride + (int64_t)gcol[u] * a.s_col_stride] = s;
    }
  }
}

// Generic kernel: any group size and alignment; one wavefront per group, two passes.
template <int XDT>
__global__ __launch_bounds__(kQuantThreads) void group_quant_generic_kernel(QuantArgs a) {
  using E = Elem<XDT>;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t gid = blockIdx.x * (kQuantThreads / 64) + (threadIdx.x >> 6);
  if (gid >= a.total_groups) return;  // whole wavefront leaves together
  const uint32_t row = gid / a.groups_per_row;
  const uint32_t gcol = gid - row * a.groups_per_row;
  const typename E::raw* xp = reinterpret_cast<const typename E::raw*>(a.x) +
                              (int64_t)row * a.x_row_stride + (int64_t)gcol * a.group_size;
  uint8_t* qp = a.q + (int64_t)row * a.q_row_stride + (int64_t)gcol * a.group_size;

  uint32_t m = 0u;
  for (uint32_t i = lane; i < a.group_size; i += 64) m = max(m, (uint32_t)xp[i] & E::kAbs);
  m = group_max_u32<64>(m);
  float amax = E::widen(m);
  if (!(amax != amax)) amax = fmaxf(amax, a.floor);
  const float s = derive_scale(amax, a);
  const float r = 1.0f / s;
  for (uint32_t i = lane; i < a.group_size; i += 64) {
    float y = quantize_value(E::widen((uint32_t)xp[i]), s, r, a, short_division_ok(m >= E::kInf, s));
    if (m >= E::kInf) y = unclamped_overflow(E::widen((uint32_t)xp[i]), s, r, y, a);
    uint32_t wd = pack2<false>(y, 0.0f, 0u, a.e5m2);
    wd = fix_nan_byte(wd, 0, y, a.e5m2);
    qp[i] = (uint8_t)(wd & 0xFFu);
  }
  if (lane == 0) a.s[(int64_t)row * a.s_row_stride + (int64_t)gcol * a.s_col_stride] = s;
}

template <int XDT>
int launch_quant(const QuantArgs& a, bool vec_ok, hipStream_t stream, bool silu = false) {
  const uint32_t g = a.group_size;
  int lpg = 0;
  if (vec_ok && g % 8 == 0) {
    uint32_t l = g / 8;
    if (l == 1 || l == 2 || l == 4 || l == 8 || l == 16 || l == 32 || l == 64) lpg = (int)l;
  }
  const int rules = (a.scale_rule == FG_SCALE_MUL_INV && a.pow2_rule == FG_POW2_NONE && !a.e5m2)
                        ? (a.quotient_rule == FG_QUOT_RECIP_MUL ? 1 : 2) : 0;
  if (silu) {
    if (lpg != 16 && lpg != 8)
      FG_FAIL(FG_ERR_UNSUPPORTED, "fused activation + quantizer: group size 64 or 128 and 16-byte aligned rows only");
    const uint64_t chunks = (uint64_t)a.total_groups * (uint64_t)lpg;
    const bool small = chunks <= kQuantSmallChunks;
    dim3 grid((uint32_t)ceil_div((int64_t)chunks, (int64_t)kQuantThreads * (small ? 1 : kQuantUnrollLarge)));
    if (lpg == 16 && rules == 2) {
      if (small) FG_LAUNCH((group_quant_vec_kernel<XDT, 16, 1, true, 2>), grid, dim3(kQuantThreads), 0, stream, a);
      else FG_LAUNCH((group_quant_vec_kernel<XDT, 16, kQuantUnrollLarge, true, 2>), grid, dim3(kQuantThreads), 0, stream, a);
    } else if (lpg == 16) {
      if (small) FG_LAUNCH((group_quant_vec_kernel<XDT, 16, 1, true>), grid, dim3(kQuantThreads), 0, stream, a);
      else FG_LAUNCH((group_quant_vec_kernel<XDT, 16, kQuantUnrollLarge, true>), grid, dim3(kQuantThreads), 0, stream, a);
    } else {
      if (small) FG_LAUNCH((group_quant_vec_kernel<XDT, 8, 1, true>), grid, dim3(kQuantThreads), 0, stream, a);
      else FG_LAUNCH((group_quant_vec_kernel<XDT, 8, kQuantUnrollLarge, true>), grid, dim3(kQuantThreads), 0, stream, a);
    }
    FG_CHECK_LAUNCH("group_quant_vec_kernel (fused activation)");
    return FG_OK;
  }
  if (lpg == 0) {
    dim3 grid((uint32_t)ceil_div(a.total_groups, kQuantThreads / 64));
    FG_LAUNCH(group_quant_generic_kernel<XDT>, grid, dim3(kQuantThreads), 0, stream, a);
    FG_CHECK_LAUNCH("group_quant_generic_kernel");
    return FG_OK;
  }
  const uint64_t chunks = (uint64_t)a.total_groups * (uint64_t)lpg;
  const bool small = chunks <= kQuantSmallChunks;
  dim3 grid((uint32_t)ceil_div((int64_t)chunks, (int64_t)kQuantThreads * (small ? 1 : kQuantUnrollLarge)));
  if (lpg == 16 && rules != 0) {  // group size 128 under either operator's default rules
    if (rules == 1) {
      if (small) FG_LAUNCH((group_quant_vec_kernel<XDT, 16, 1, false, 1>), grid, dim3(kQuantThreads), 0, stream, a);
      else FG_LAUNCH((group_quant_vec_kernel<XDT, 16, kQuantUnrollLarge, false, 1>), grid, dim3(kQuantThreads), 0, stream, a);
    } else {
      if (small) FG_LAUNCH((group_quant_vec_kernel<XDT, 16, 1, false, 2>), grid, dim3(kQuantThreads), 0, stream, a);
      else FG_LAUNCH((group_quant_vec_kernel<XDT, 16, kQuantUnrollLarge, false, 2>), grid, dim3(kQuantThreads), 0, stream, a);
    }
    FG_CHECK_LAUNCH("group_quant_vec_kernel");
    return FG_OK;
  }
  switch (lpg) {
#define FG_CASE(L)                                                                                                       \
  case L:                                                                                                                \
    if (small) FG_LAUNCH((group_quant_vec_kernel<XDT, L, 1>), grid, dim3(kQuantThreads), 0, stream, a);         \
    else FG_LAUNCH((group_quant_vec_kernel<XDT, L, kQuantUnrollLarge>), grid, dim3(kQuantThreads), 0, stream, a); \
    break;
    FG_CASE(1) FG_CASE(2) FG_CASE(4) FG_CASE(8) FG_CASE(16) FG_CASE(32) FG_CASE(64)
#undef FG_CASE
  }
  FG_CHECK_LAUNCH("group_quant_vec_kernel");
  return FG_OK;
}

// ---- 128 x 128 block quantizer (weights)
//
// One workgroup per block: thread t owns the 8-element chunk (t & 15) of rows (t >> 4) + 16 i, i < 8, so a
// wavefront reads four whole 256-byte (bf16) row pieces per load instruction.  The block's absolute maximum goes
// through DPP within a wavefront and through LDS across the four; scale and codes follow the group
// quantizer's rules.  Elements past the matrix edge count as zeros (the reference pads with zeros,
// tests/test_fp8_einsum.py:89-103) and are not written.
constexpr int kBlockQuantEdge = 128;

struct BlockQuantArgs {
  QuantArgs r;         // pointers, row strides, rules; group fields unused
  uint32_t rows, cols;
  int vec;             // rows of x are 16-byte aligned and rows of q 8-byte aligned
};

template <int XDT>
__global__ __launch_bounds__(kQuantThreads) void block_quant_kernel(BlockQuantArgs b) {
  using E = Elem<XDT>;
  using Raw = typename E::raw;
  constexpr int kWords = sizeof(Raw) * 8 / 4;
  constexpr int kIters = kBlockQuantEdge * kBlockQuantEdge / 8 / kQuantThreads;  // 8
  __shared__ uint32_t wave_max[kQuantThreads / 64];
  const QuantArgs& a = b.r;
  const uint32_t t = threadIdx.x;
  const uint32_t col = blockIdx.x * kBlockQuantEdge + (t & 15u) * 8u;
  const uint32_t row0 = blockIdx.y * kBlockQuantEdge + (t >> 4);
  const bool whole = b.vec && col + 8u <= b.cols;  // the chunk lies inside the row and takes vector accesses

  uint32_t w[kIters][kWords];
#pragma unroll
  for (int i = 0; i < kIters; ++i) {
    const uint32_t row = row0 + 16u * (uint32_t)i;
#pragma unroll
    for (int k = 0; k < kWords; ++k) w[i][k] = 0u;
    if (row < b.rows && col < b.cols) {
      const Raw* p = reinterpret_cast<const Raw*>(a.x) + (int64_t)row * a.x_row_stride + col;
      if (whole) {
        const u32x4* p4 = reinterpret_cast<const u32x4*>(p);
        u32x4 v = p4[0];
        w[i][0] = v.x; w[i][1] = v.y; w[i][2] = v.z; w[i][3] = v.w;
        if constexpr (kWords == 8) {
          u32x4 v2 = p4[1];
          w[i][4] = v2.x; w[i][5] = v2.y; w[i][6] = v2.z; w[i][7] = v2.w;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t v = (col + (uint32_t)e < b.cols) ? (uint32_t)p[e] : 0u;
          if constexpr (kWords == 4) w[i][e >> 1] |= v << (16 * (e & 1));
          else w[i][e] = v;
        }
      }
    }
  }

  // absolute maximum on the raw bit patterns: NaN patterns compare above everything
  uint32_t m = 0u;
#pragma unroll
  for (int i = 0; i < kIters; ++i)
#pragma unroll
    for (int k = 0; k < kWords; ++k) {
      if constexpr (kWords == 4) m = max(m, max(w[i][k] & E::kAbs, (w[i][k] >> 16) & E::kAbs));
      else m = max(m, w[i][k] & E::kAbs);
    }
  m = group_max_u32<64>(m);
  if ((t & 63u) == 0u) wave_max[t >> 6] = m;
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kQuantThreads / 64; ++k) m = max(m, wave_max[k]);

  float amax = E::widen(m);
  const bool special = m >= E::kInf;  // Inf or NaN somewhere in the block
  if (!(amax != amax)) amax = fmaxf(amax, a.floor);
  const float s = derive_scale(amax, a);
  const float r = 1.0f / s;
  if (t == 0) a.s[(int64_t)blockIdx.y * a.s_row_stride + (int64_t)blockIdx.x * a.s_col_stride] = s;

#pragma unroll
  for (int i = 0; i < kIters; ++i) {
    const uint32_t row = row0 + 16u * (uint32_t)i;
    if (!(row < b.rows && col < b.cols)) continue;
    float y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float xv;
      if constexpr (kWords == 4) xv = E::widen((w[i][e >> 1] >> (16 * (e & 1))) & 0xFFFFu);
      else xv = E::widen(w[i][e]);
      y[e] = quantize_value(xv, s, r, a, short_division_ok(special, s));
      if (special) y[e] = unclamped_overflow(xv, s, r, y[e], a);
    }
    uint32_t w0 = pack2<false>(y[0], y[1], 0u, a.e5m2);
    w0 = pack2<true>(y[2], y[3], w0, a.e5m2);
    uint32_t w1 = pack2<false>(y[4], y[5], 0u, a.e5m2);
    w1 = pack2<true>(y[6], y[7], w1, a.e5m2);
    if (special || !(s == s)) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        w0 = fix_nan_byte(w0, e, y[e], a.e5m2);
        w1 = fix_nan_byte(w1, e, y[4 + e], a.e5m2);
      }
    }
    uint8_t* qp = a.q + (int64_t)row * a.q_row_stride + col;
    if (whole) {
      u32x2 out = {w0, w1};
      *reinterpret_cast<u32x2*>(qp) = out;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (col + (uint32_t)e < b.cols) qp[e] = (uint8_t)(((e < 4 ? w0 : w1) >> (8 * (e & 3))) & 0xFFu);
    }
  }
}

}  // namespace
}  // namespace fg

extern "C" int fg_block_quant_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride,
                                  void* q, int q_dtype, int64_t q_row_stride,
                                  float* s, int64_t s_row_stride, int64_t s_col_stride,
                                  int64_t block_rows, int64_t block_cols, float amax_floor, float fp8_min, float fp8_max,
                                  float inv_fp8_max, int scale_rule, int quotient_rule, int pow2_rule,
                                  void* stream) {
  using namespace fg;
  const char* const who = "fg_block_quant_fp8";
  if (rows < 0 || cols < 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: negative size", who);
  if (rows == 0 || cols == 0) return FG_OK;
  if (!x || !q || !s) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null pointer", who);
  if (block_rows != kBlockQuantEdge || block_cols != kBlockQuantEdge)
    FG_FAIL(FG_ERR_UNSUPPORTED, "%s: only 128 x 128 blocks are implemented (got %lld x %lld)", who,
            (long long)block_rows, (long long)block_cols);
  if (x_dtype != FG_BF16 && x_dtype != FG_F16 && x_dtype != FG_F32) FG_FAIL(FG_ERR_INVALID_ARG, "%s: x_dtype %d", who, x_dtype);
  if (q_dtype != FG_FP8_E4M3FN && q_dtype != FG_FP8_E5M2) FG_FAIL(FG_ERR_INVALID_ARG, "%s: q_dtype %d", who, q_dtype);
  if (scale_rule < 0 || scale_rule > 1 || quotient_rule < 0 || quotient_rule > 1 || pow2_rule < 0 || pow2_rule > 3)
    FG_FAIL(FG_ERR_INVALID_ARG, "%s: bad rule selector", who);
  if (x_row_stride < cols || q_row_stride < cols) FG_FAIL(FG_ERR_INVALID_ARG, "%s: row stride smaller than cols", who);
  const int64_t block_rows_n = ceil_div(rows, (int64_t)kBlockQuantEdge), block_cols_n = ceil_div(cols, (int64_t)kBlockQuantEdge);
  if (block_rows_n > 65535 || block_cols_n > 0x7FFFFFFF || cols > 0x7FFFFF00ll)
    FG_FAIL(FG_ERR_UNSUPPORTED, "%s: more than 65535 block rows or 2^31 columns", who);
  const size_t esz = (x_dtype == FG_F32) ? 4 : 2;
  BlockQuantArgs b = {};
  b.r.x = x; b.r.q = (uint8_t*)q; b.r.s = s;
  b.r.x_row_stride = x_row_stride; b.r.q_row_stride = q_row_stride;
  b.r.s_row_stride = s_row_stride; b.r.s_col_stride = s_col_stride;
  b.r.floor = amax_floor; b.r.lo = fp8_min; b.r.hi = fp8_max; b.r.inv_max = inv_fp8_max;
  b.r.scale_rule = scale_rule; b.r.quotient_rule = quotient_rule; b.r.pow2_rule = pow2_rule;
  b.r.e5m2 = (q_dtype == FG_FP8_E5M2);
  b.rows = (uint32_t)rows; b.cols = (uint32_t)cols;
  b.vec = ((uintptr_t)x % 16 == 0) && ((x_row_stride * esz) % 16 == 0) && ((uintptr_t)q % 8 == 0) && (q_row_stride % 8 == 0);
  const dim3 grid((uint32_t)block_cols_n, (uint32_t)block_rows_n);
  if (x_dtype == FG_BF16) FG_LAUNCH(block_quant_kernel<FG_BF16>, grid, dim3(kQuantThreads), 0, (hipStream_t)stream, b);
  else if (x_dtype == FG_F16) FG_LAUNCH(block_quant_kernel<FG_F16>, grid, dim3(kQuantThreads), 0, (hipStream_t)stream, b);
  else FG_LAUNCH(block_quant_kernel<FG_F32>, grid, dim3(kQuantThreads), 0, (hipStream_t)stream, b);
  FG_CHECK_LAUNCH("block_quant_kernel");
  return FG_OK;
}

namespace fg {
namespace {
// silu: the quantized value is silu(x[r, c]) * x[r, c + up_offset] (x then has at least up_offset + cols columns)
int group_quant_entry(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride,
                      void* q, int q_dtype, int64_t q_row_stride,
                      float* s, int64_t s_row_stride, int64_t s_col_stride,
                      int64_t group_size, float amax_floor, float fp8_min, float fp8_max,
                      float inv_fp8_max, int scale_rule, int quotient_rule, int pow2_rule,
                      void* stream, bool silu, int64_t up_offset) {
  if (rows < 0 || cols < 0) FG_FAIL(FG_ERR_INVALID_ARG, "fg_group_quant_fp8: negative size");
  if (rows == 0 || cols == 0) return FG_OK;
  if (!x || !q || !s) FG_FAIL(FG_ERR_INVALID_ARG, "fg_group_quant_fp8: null pointer");
  if (group_size <= 0 || cols % group_size != 0)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_group_quant_fp8: cols %lld not divisible by group_size %lld",
            (long long)cols, (long long)group_size);
  if (x_dtype != FG_BF16 && x_dtype != FG_F16 && x_dtype != FG_F32)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_group_quant_fp8: x_dtype %d", x_dtype);
  if (q_dtype != FG_FP8_E4M3FN && q_dtype != FG_FP8_E5M2)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_group_quant_fp8: q_dtype %d", q_dtype);
  if (scale_rule < 0 || scale_rule > 1 || quotient_rule < 0 || quotient_rule > 1 || pow2_rule < 0 || pow2_rule > 3)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_group_quant_fp8: bad rule selector");
  if (x_row_stride < cols || q_row_stride < cols)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_group_quant_fp8: row stride smaller than cols");
  if (silu && (up_offset < cols || x_row_stride < up_offset + cols))
    FG_FAIL(FG_ERR_INVALID_ARG, "fused activation + quantizer: the up half must follow the gate half inside the row");
  if (group_size > (int64_t)1 << 24) FG_FAIL(FG_ERR_UNSUPPORTED, "fg_group_quant_fp8: group_size too large");

  const int64_t groups_per_row = cols / group_size;
  if (groups_per_row > 0x7FFFFFFF) FG_FAIL(FG_ERR_UNSUPPORTED, "fg_group_quant_fp8: too many groups per row");
  const size_t esz = (x_dtype == FG_F32) ? 4 : 2;
  const bool vec_ok = ((uintptr_t)x % 16 == 0) && ((x_row_stride * esz) % 16 == 0) &&
                      ((uintptr_t)q % 8 == 0) && (q_row_stride % 8 == 0) && (!silu || (up_offset * esz) % 16 == 0);

  // Launch in row slabs so that 32-bit chunk indices cannot overflow.
  const int64_t max_groups = (int64_t)1 << 24;
  int64_t rows_per_launch = max_groups / groups_per_row;
  if (rows_per_launch < 1) rows_per_launch = 1;
  for (int64_t r0 = 0; r0 < rows; r0 += rows_per_launch) {
    const int64_t nr = (rows - r0 < rows_per_launch) ? rows - r0 : rows_per_launch;
    QuantArgs a;
    a.x = (const char*)x + r0 * x_row_stride * (int64_t)esz;
    a.q = (uint8_t*)q + r0 * q_row_stride;
    a.s = s + r0 * s_row_stride;
    a.x_row_stride = x_row_stride;
    a.q_row_stride = q_row_stride;
    a.s_row_stride = s_row_stride;
    a.s_col_stride = s_col_stride;
    a.groups_per_row = (uint32_t)groups_per_row;
    a.total_groups = (uint32_t)(nr * groups_per_row);
    a.group_size = (uint32_t)group_size;
    a.floor = amax_floor;
    a.lo = fp8_min;
    a.hi = fp8_max;
    a.inv_max = inv_fp8_max;
    a.scale_rule = scale_rule;
    a.quotient_rule = quotient_rule;
    a.pow2_rule = pow2_rule;
    a.e5m2 = (q_dtype == FG_FP8_E5M2);
    a.up_offset = up_offset;
    a.inv_groups_per_row = nr == 1 ? 0.0f : 1.0f / (float)groups_per_row;  // nr > 1 implies fewer than 2^24 groups in all
    int rc;
    if (x_dtype == FG_BF16) rc = launch_quant<FG_BF16>(a, vec_ok, (hipStream_t)stream, silu);
    else if (x_dtype == FG_F16) rc = launch_quant<FG_F16>(a, vec_ok, (hipStream_t)stream, silu);
    else rc = launch_quant<FG_F32>(a, vec_ok, (hipStream_t)stream, silu);
    if (rc != FG_OK) return rc;
  }
  return FG_OK;
}

// out[r, c] = silu(x[r, c]) * x[r, c + up_offset] rounded to x's type; eight elements per thread
template <int XDT>
__global__ __launch_bounds__(kQuantThreads) void silu_mul_kernel(const void* x, void* out, int64_t x_row_stride,
                                                                 int64_t out_row_stride, int64_t up_offset,
                                                                 uint32_t chunks_per_row, uint32_t total_chunks) {
  using E = Elem<XDT>;
  using Raw = typename E::raw;
  constexpr int kWords = sizeof(Raw) * 8 / 4;
  const uint32_t c = blockIdx.x * kQuantThreads + threadIdx.x;
  if (c >= total_chunks) return;
  const uint32_t row = c / chunks_per_row, col = (c - row * chunks_per_row) * 8u;
  const Raw* p = reinterpret_cast<const Raw*>(x) + (int64_t)row * x_row_stride + col;
  uint32_t w[kWords], up[kWords];
#pragma unroll
  for (int k = 0; k < kWords / 4; ++k) {
    const u32x4 v = reinterpret_cast<const u32x4*>(p)[k], t = reinterpret_cast<const u32x4*>(p + up_offset)[k];
    w[4 * k] = v.x; w[4 * k + 1] = v.y; w[4 * k + 2] = v.z; w[4 * k + 3] = v.w;
    up[4 * k] = t.x; up[4 * k + 1] = t.y; up[4 * k + 2] = t.z; up[4 * k + 3] = t.w;
  }
  silu_mul_words<XDT, kWords>(w, up);
  Raw* o = reinterpret_cast<Raw*>(out) + (int64_t)row * out_row_stride + col;
#pragma unroll
  for (int k = 0; k < kWords / 4; ++k) {
    const u32x4 v = {w[4 * k], w[4 * k + 1], w[4 * k + 2], w[4 * k + 3]};
    reinterpret_cast<u32x4*>(o)[k] = v;
  }
}
}  // namespace
}  // namespace fg

extern "C" int fg_group_quant_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride,
                                  void* q, int q_dtype, int64_t q_row_stride,
                                  float* s, int64_t s_row_stride, int64_t s_col_stride,
                                  int64_t group_size, float amax_floor, float fp8_min, float fp8_max,
                                  float inv_fp8_max, int scale_rule, int quotient_rule, int pow2_rule,
                                  void* stream) {
  return fg::group_quant_entry(x, x_dtype, rows, cols, x_row_stride, q, q_dtype, q_row_stride, s, s_row_stride,
                               s_col_stride, group_size, amax_floor, fp8_min, fp8_max, inv_fp8_max, scale_rule,
                               quotient_rule, pow2_rule, stream, false, 0);
}

extern "C" int fg_silu_mul_group_quant_fp8(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride,
                                           int64_t up_offset, void* q, int q_dtype, int64_t q_row_stride,
                                           float* s, int64_t s_row_stride, int64_t s_col_stride,
                                           int64_t group_size, float amax_floor, float fp8_min, float fp8_max,
                                           float inv_fp8_max, int scale_rule, int quotient_rule, int pow2_rule,
                                           void* stream) {
  return fg::group_quant_entry(x, x_dtype, rows, cols, x_row_stride, q, q_dtype, q_row_stride, s, s_row_stride,
                               s_col_stride, group_size, amax_floor, fp8_min, fp8_max, inv_fp8_max, scale_rule,
                               quotient_rule, pow2_rule, stream, true, up_offset);
}

extern "C" int fg_silu_mul(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t x_row_stride, int64_t up_offset,
                           void* out, int64_t out_row_stride, void* stream) {
  using namespace fg;
  if (rows < 0 || cols < 0) FG_FAIL(FG_ERR_INVALID_ARG, "fg_silu_mul: negative size");
  if (rows == 0 || cols == 0) return FG_OK;
  if (!x || !out) FG_FAIL(FG_ERR_INVALID_ARG, "fg_silu_mul: null pointer");
  if (x_dtype != FG_BF16 && x_dtype != FG_F16 && x_dtype != FG_F32) FG_FAIL(FG_ERR_INVALID_ARG, "fg_silu_mul: x_dtype %d", x_dtype);
  if (up_offset < cols || x_row_stride < up_offset + cols || out_row_stride < cols)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_silu_mul: the up half must follow the gate half inside the row");
  const int64_t esz = (x_dtype == FG_F32) ? 4 : 2;
  if (cols % 8 != 0 || (uintptr_t)x % 16 != 0 || (uintptr_t)out % 16 != 0 || (x_row_stride * esz) % 16 != 0 ||
      (out_row_stride * esz) % 16 != 0 || (up_offset * esz) % 16 != 0)
    FG_FAIL(FG_ERR_UNSUPPORTED, "fg_silu_mul: rows and halves must be 16-byte aligned and cols a multiple of 8");
  const int64_t chunks = rows * (cols / 8);
  if (chunks > 0x7FFFFFFF) FG_FAIL(FG_ERR_UNSUPPORTED, "fg_silu_mul: more than 2^31 chunks");
  const dim3 grid((uint32_t)ceil_div(chunks, (int64_t)kQuantThreads));
  const uint32_t cpr = (uint32_t)(cols / 8), total = (uint32_t)chunks;
  if (x_dtype == FG_BF16) FG_LAUNCH(silu_mul_kernel<FG_BF16>, grid, dim3(kQuantThreads), 0, (hipStream_t)stream, x, out, x_row_stride, out_row_stride, up_offset, cpr, total);
  else if (x_dtype == FG_F16) FG_LAUNCH(silu_mul_kernel<FG_F16>, grid, dim3(kQuantThreads), 0, (hipStream_t)stream, x, out, x_row_stride, out_row_stride, up_offset, cpr, total);
  else FG_LAUNCH(silu_mul_kernel<FG_F32>, grid, dim3(kQuantThreads), 0, (hipStream_t)stream, x, out, x_row_stride, out_row_stride, up_offset, cpr, total);
  FG_CHECK_LAUNCH("silu_mul_kernel");
  return FG_OK;
}


extern "C" int fg_act_quant_bf16(const void* x, void* y, float* s, int64_t rows, int64_t cols,
                                 int64_t block_size, int round_scale, void* stream) {
  if (block_size <= 0 || cols % (block_size > 0 ? block_size : 1) != 0) {
    snprintf(fg::error_buffer(), fg::kErrorBufferBytes,
             "fg_act_quant_bf16: last dimension %lld must be divisible by block_size %lld",
             (long long)cols, (long long)block_size);
    return FG_ERR_INVALID_ARG;
  }
  return fg_group_quant_fp8(x, FG_BF16, rows, cols, cols, y, FG_FP8_E4M3FN, cols, s, cols / block_size, 1,
                            block_size, 1e-4f, -448.0f, 448.0f, 1.0f / 448.0f, FG_SCALE_MUL_INV,
                            FG_QUOT_RECIP_MUL, round_scale ? FG_POW2_BITS : FG_POW2_NONE, stream);
}
