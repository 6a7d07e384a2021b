// Sum over the top-k slots of every token: out[t, :] = sum_k in[t, k, :], the last step of an expert layer.
//
// Follows moe_sum_kernel of the reference (src/flag_gems/fused/moe_sum.py:34-67): an fp32 running sum over the
// slots in slot order, one rounding to the output type.  HBM bound: (top_k + 1) * element size bytes per output
// element; a lane owns eight consecutive elements (one 16-byte load per slot for 16-bit types).

#include "fg_common.h"

namespace fg {
namespace {

constexpr int kSumThreads = 256;

__device__ __forceinline__ float bf16_bits_to_float(uint32_t h) { return bits_to_float(h << 16); }
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
  // round to nearest even; NaN stays NaN
  const uint32_t u = float_to_bits(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// DT: FG_BF16, FG_F16 or FG_F32.  chunks_per_row = hidden / 8; strides in elements.
template <int DT>
__global__ __launch_bounds__(kSumThreads) void moe_sum_kernel(const void* __restrict__ in, void* __restrict__ out, int top_k,
                                                              int64_t in_token_stride, int64_t in_slot_stride,
                                                              int64_t out_token_stride, uint32_t chunks_per_row, uint32_t total) {
  const uint32_t c = blockIdx.x * kSumThreads + threadIdx.x;
  if (c >= total) return;
  const uint32_t t = c / chunks_per_row, h = (c - t * chunks_per_row) * 8;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (DT == FG_F32) {
    const float* p = reinterpret_cast<const float*>(in) + (int64_t)t * in_token_stride + h;
    for (int k = 0; k < top_k; ++k, p += in_slot_stride) {
      const v4f a = *reinterpret_cast<const v4f*>(p), b = *reinterpret_cast<const v4f*>(p + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { acc[e] += a[e]; acc[4 + e] += b[e]; }
    }
    float* q = reinterpret_cast<float*>(out) + (int64_t)t * out_token_stride + h;
    *reinterpret_cast<v4f*>(q) = v4f{acc[0], acc[1], acc[2], acc[3]};
    *reinterpret_cast<v4f*>(q + 4) = v4f{acc[4], acc[5], acc[6], acc[7]};
    return;
  }
  const uint16_t* p = reinterpret_cast<const uint16_t*>(in) + (int64_t)t * in_token_stride + h;
  for (int k = 0; k < top_k; ++k, p += in_slot_stride) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(p);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (DT == FG_BF16) {
        acc[2 * e] += bf16_bits_to_float(w[e] & 0xFFFFu);
        acc[2 * e + 1] += bf16_bits_to_float(w[e] >> 16);
      } else {
        acc[2 * e] += (float)__builtin_bit_cast(_Float16, (uint16_t)(w[e] & 0xFFFFu));
        acc[2 * e + 1] += (float)__builtin_bit_cast(_Float16, (uint16_t)(w[e] >> 16));
      }
    }
  }
  uint32_t r[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (DT == FG_BF16) {
      r[e] = float_to_bf16_bits(acc[2 * e]) | (float_to_bf16_bits(acc[2 * e + 1]) << 16);
    } else {
      r[e] = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)acc[2 * e]) |
             ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)acc[2 * e + 1]) << 16);
    }
  }
  *reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(out) + (int64_t)t * out_token_stride + h) = u32x4{r[0], r[1], r[2], r[3]};
}

}  // namespace
}  // namespace fg

extern "C" int fg_moe_sum(const void* in, int dtype, int64_t tokens, int64_t top_k, int64_t hidden, int64_t in_token_stride,
                          int64_t in_slot_stride, void* out, int64_t out_token_stride, void* stream) {
  using namespace fg;
  if (tokens < 0 || top_k < 0 || hidden < 0) FG_FAIL(FG_ERR_INVALID_ARG, "fg_moe_sum: negative size");
  if (tokens == 0 || hidden == 0) return FG_OK;
  if (!in || !out) FG_FAIL(FG_ERR_INVALID_ARG, "fg_moe_sum: null pointer");
  if (dtype != FG_BF16 && dtype != FG_F16 && dtype != FG_F32) FG_FAIL(FG_ERR_INVALID_ARG, "fg_moe_sum: dtype %d", dtype);
  if (top_k > 0x7FFFFFFF) FG_FAIL(FG_ERR_INVALID_ARG, "fg_moe_sum: top_k %lld", (long long)top_k);
  const int64_t esz = dtype == FG_F32 ? 4 : 2;
  if (hidden % 8 != 0 || (uintptr_t)in % 16 != 0 || (uintptr_t)out % 16 != 0 || (in_token_stride * esz) % 16 != 0 ||
      (in_slot_stride * esz) % 16 != 0 || (out_token_stride * esz) % 16 != 0)
    FG_FAIL(FG_ERR_UNSUPPORTED, "fg_moe_sum: rows must be 16-byte aligned and hidden a multiple of 8");
  const int64_t chunks = tokens * (hidden / 8);
  if (chunks > 0x7FFFFFFF) FG_FAIL(FG_ERR_UNSUPPORTED, "fg_moe_sum: more than 2^31 chunks");
  const dim3 grid((uint32_t)ceil_div(chunks, (int64_t)kSumThreads));
  const uint32_t cpr = (uint32_t)(hidden / 8), total = (uint32_t)chunks;
  if (dtype == FG_BF16) FG_LAUNCH(moe_sum_kernel<FG_BF16>, grid, dim3(kSumThreads), 0, (hipStream_t)stream, in, out, (int)top_k, in_token_stride, in_slot_stride, out_token_stride, cpr, total);
  else if (dtype == FG_F16) FG_LAUNCH(moe_sum_kernel<FG_F16>, grid, dim3(kSumThreads), 0, (hipStream_t)stream, in, out, (int)top_k, in_token_stride, in_slot_stride, out_token_stride, cpr, total);
  else FG_LAUNCH(moe_sum_kernel<FG_F32>, grid, dim3(kSumThreads), 0, (hipStream_t)stream, in, out, (int)top_k, in_token_stride, in_slot_stride, out_token_stride, cpr, total);
  FG_CHECK_LAUNCH("moe_sum_kernel");
  return FG_OK;
}
