// Device-side pieces of the FP8 group quantizer shared by the kernels that produce quantized activations:
// element types, the scale rules, the division, the fp8 packing and the across-lane maximum.
#pragma once

#include "fg_common.h"

namespace fg {
namespace {

struct QuantArgs {
  const void* x;
  uint8_t* q;
  float* s;
  int64_t x_row_stride, q_row_stride, s_row_stride, s_col_stride;
  uint32_t groups_per_row;
  uint32_t total_groups;
  uint32_t group_size;
  float floor, lo, hi, inv_max;
  int scale_rule, quotient_rule, pow2_rule, e5m2;
  int64_t up_offset;  // fused SiLU-and-mul producer: elements from a gate value to its up value (same row)
  float inv_groups_per_row;  // fp32(1 / groups_per_row), or 0 when the launch covers a single row
};

// n / d for n < 2^24 and 1 <= d < 2^24, given inv = fp32(1 / d): the fp32 product is within one of the quotient
// ((n / d) 2^-23 < 1 for d >= 2, exact for d = 1), and one step either way from the remainder makes it exact.
// With inv = 0 and n < d the result is 0 whatever d is.  About ten instructions where the compiler's 32-bit
// division takes about thirty, once per 8-element chunk.
__device__ __forceinline__ uint32_t divide_below_2_24(uint32_t n, uint32_t d, float inv, uint32_t& remainder) {
  uint32_t q = (uint32_t)((float)n * inv);
  int32_t r = (int32_t)(n - q * d);
  if (r < 0) { q -= 1u; r += (int32_t)d; }
  else if ((uint32_t)r >= d) { q += 1u; r -= (int32_t)d; }
  remainder = (uint32_t)r;
  return q;
}

template <int XDT> struct Elem;
template <> struct Elem<FG_BF16> {
  using raw = uint16_t;
  static constexpr uint32_t kAbs = 0x7FFFu, kInf = 0x7F80u;
  __device__ static float widen(uint32_t b) { return bits_to_float(b << 16); }
  // two values -> two bf16 in one word, round to nearest even (one v_cvt_pk_bf16_f32; NaN stays NaN)
  __device__ static uint32_t narrow2(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
  }
};
template <> struct Elem<FG_F16> {
  using raw = uint16_t;
  static constexpr uint32_t kAbs = 0x7FFFu, kInf = 0x7C00u;
  __device__ static float widen(uint32_t b) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
  }
  __device__ static uint32_t narrow2(float lo, float hi) {
    // The empty statement pins both values in registers as fp32 numbers: without it the compiler folds the
    // multiplication that produced them into the conversion (v_fma_mixlo_f16), which rounds the exact product to
    // fp16 once instead of to fp32 and then to fp16 and lands on the other neighbour about once in 10^4 values.
    asm("" : "+v"(lo), "+v"(hi));
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lo) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
  }
};
template <> struct Elem<FG_F32> {
  using raw = uint32_t;
  static constexpr uint32_t kAbs = 0x7FFFFFFFu, kInf = 0x7F800000u;
  __device__ static float widen(uint32_t b) { return bits_to_float(b); }
};

// gate * sigmoid(gate) * up in fp32, as the reference's activation kernel computes it
// (src/flag_gems/fused/fused_moe.py:795-800: x / (1 + exp(-x)) * y), rounded once to the input's type.
template <int XDT>
__device__ __forceinline__ float silu_mul_f32(uint32_t gate, uint32_t up) {
  using E = Elem<XDT>;
  const float g = E::widen(gate), u = E::widen(up);
  if constexpr (XDT == FG_F32) return g / (1.0f + expf(-g)) * u;
  // 16-bit results: the hardware exponential and reciprocal (what the reference's tl.exp and tl.fdiv compile to)
  // are wrong by a few fp32 steps, thousands of times below the step of the result; the correctly rounded
  // routines cost more instructions than the rest of the quantizer together and would bind the kernel.
  return __fdividef(g, 1.0f + __expf(-g)) * u;
}

// eight gate values and eight up values (raw words as loaded) -> eight activated values in the same packing
template <int XDT, int WORDS>
__device__ __forceinline__ void silu_mul_words(uint32_t (&w)[WORDS], const uint32_t (&up)[WORDS]) {
#pragma unroll
  for (int i = 0; i < WORDS; ++i) {
    if constexpr (WORDS == 4) {
      w[i] = Elem<XDT>::narrow2(silu_mul_f32<XDT>(w[i] & 0xFFFFu, up[i] & 0xFFFFu), silu_mul_f32<XDT>(w[i] >> 16, up[i] >> 16));
    } else {
      w[i] = float_to_bits(silu_mul_f32<XDT>(w[i], up[i]));
    }
  }
}

// scale from the group's absolute maximum (already floored), following the requested rules
__device__ __forceinline__ float derive_scale(float amax, const QuantArgs& a) {
  float s = (a.scale_rule == FG_SCALE_MUL_INV) ? amax * a.inv_max : amax / a.hi;
  if (a.pow2_rule == FG_POW2_BITS) {
    // exponent + (mantissa != 0) re-assembled with 32-bit wrap-around
    // (reference src/flag_gems/fused/act_quant.py:22-41)
    uint32_t b = float_to_bits(s);
    uint32_t e = (b >> 23) & 0xFFu;
    uint32_t m = b & 0x7FFFFFu;
    uint32_t l = e - 127u + (m != 0u ? 1u : 0u);
    s = bits_to_float((l + 127u) << 23);
  } else if (a.pow2_rule == FG_POW2_BITS_CLAMPED) {
    // the same on |s| with the exponent field held in [1, 254] (reference tests/test_fp8_einsum.py:63-67)
    const uint32_t b = float_to_bits(s) & 0x7FFFFFFFu;
    uint32_t e = (b >> 23) + ((b & 0x7FFFFFu) != 0u ? 1u : 0u);
    e = e < 1u ? 1u : (e > 254u ? 254u : e);
    s = bits_to_float(e << 23);
  } else if (a.pow2_rule == FG_POW2_LOG2) {
    // exp2(ceil(log2(max(|s|, 1e-10)))) with log2 rounded to fp32 the way a correctly rounded
    // libm does it (reference src/flag_gems/ops/per_token_group_quant_fp8.py:65-66)
    float t = fmaxf(fabsf(s), 1e-10f);
    if (s != s) {
      // NaN stays NaN
    } else if (t < __builtin_huge_valf()) {
      // t = 2^n (1 + m 2^-23), n >= -34.  The fp32 logarithm of a t just above 2^n rounds to n itself, and the
      // ceiling then stays at n: that happens while log2(1 + m 2^-23) is below half the distance from n to the
      // next fp32 above it, 2^(j - 24) with j = floor(log2 |n|) (one less where n is minus a power of two: the
      // floats get denser on that side), i.e. for m <= floor(ln 2 * 2^(j - 1)) = 0, 0, 1, 2, 5, 11, 22 for
      // j = 0 .. 6 (the quotients are 0.35, 0.69, 1.39, 2.77, 5.55, 11.09, 22.18: none is near an integer, and the
      // second-order term of the logarithm is a millionth of them).  No logarithm is evaluated: the double
      // precision routine that was here cost as much as the rest of the quantizer together.
      const uint32_t b = float_to_bits(t);
      const int n = (int)(b >> 23) - 127;
      const uint32_t m = b & 0x7FFFFFu;
      uint32_t keep = 0;  // largest m whose logarithm still rounds to n
      if (n != 0) {
        const uint32_t an = (uint32_t)(n < 0 ? -n : n);
        int j = 31 - __builtin_clz(an);
        if (n < 0 && (an & (an - 1u)) == 0u) --j;
        keep = j < 2 ? 0u : (uint32_t)(0.69314718f * (float)(1u << (j - 1)));
      }
      const int k = n + (m > keep ? 1 : 0);
      s = bits_to_float((uint32_t)(k + 127) << 23);
    } else {
      s = t;
    }
  }
  return s;
}

// Whether x / s may be computed as below for every x of a group with scale s: no Inf or NaN in the group, and s
// far enough from the ends of the exponent range that neither r = 1 / s nor the remainder goes subnormal.
__device__ __forceinline__ bool short_division_ok(bool special, float s) {
  return !special && s >= 0x1p-60f && s <= 0x1p100f;
}

// x / s, correctly rounded, in three operations given the correctly rounded reciprocal r = RN(1 / s)
// (Markstein's sequence): q0 = RN(x r) is within a step of the quotient, the remainder e = x - q0 s is exact in
// one fused multiply-add, and RN(q0 + e r) is the correctly rounded quotient.  With s in [2^-60, 2^100] every
// quotient that can produce a non-zero fp8 code (|y| >= 2^-20) has a normal remainder; below that the last bit may
// differ from the division instruction sequence's, the code is a zero either way, and its sign is x's.
// The full sequence (v_div_scale, v_rcp, four fmas, v_div_fmas, v_div_fixup per element) made the quantizer
// VALU-bound: 115 us against 69 us with a reciprocal multiply on bf16 [8192, 14336].
__device__ __forceinline__ float short_division(float x, float s, float r) {
  const float q0 = x * r;
  const float e = __builtin_fmaf(-q0, s, x);
  const float q1 = __builtin_fmaf(e, r, q0);
  return bits_to_float((float_to_bits(q1) & 0x7FFFFFFFu) | (float_to_bits(x) & 0x80000000u));
}

__device__ __forceinline__ float quantize_value(float x, float s, float r, const QuantArgs& a, bool short_div = false) {
  float y = (a.quotient_rule == FG_QUOT_RECIP_MUL) ? x * r : (short_div ? short_division(x, s, r) : x / s);
  // clamp that lets NaN through, as torch.clamp does
  float c = fminf(fmaxf(y, a.lo), a.hi);
  return (y != y) ? y : c;
}

// The reference helpers that round scales with FG_POW2_BITS_CLAMPED cast the quotient without clamping it
// (tests/test_fp8_einsum.py:70-103), and an e4m3fn cast has no infinity: what lies past the last finite code's
// rounding interval (|y| > 464) becomes NaN.  Only an infinite input under a scale held at 2^127 gets there, so the
// callers apply this to groups that hold an Inf or NaN only.
__device__ __forceinline__ float unclamped_overflow(float x, float s, float r, float y, const QuantArgs& a) {
  if (a.pow2_rule != FG_POW2_BITS_CLAMPED || a.e5m2) return y;
  const float raw = (a.quotient_rule == FG_QUOT_RECIP_MUL) ? x * r : x / s;
  return fabsf(raw) > 464.0f ? bits_to_float(0x7FC00000u | (float_to_bits(raw) & 0x80000000u)) : y;
}

template <bool HI>
__device__ __forceinline__ uint32_t pack2(float v0, float v1, uint32_t old, int e5m2) {
  if (e5m2) return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(v0, v1, (int)old, HI);
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(v0, v1, (int)old, HI);
}

// NaN keeps its sign and takes the all-ones magnitude, whatever the converter does with it
__device__ __forceinline__ uint32_t fix_nan_byte(uint32_t word, int byte, float v, int e5m2) {
  if (v != v) {
    uint32_t code = ((float_to_bits(v) >> 24) & 0x80u) | (e5m2 ? 0x7Fu : 0x7Fu);
    word = (word & ~(0xFFu << (8 * byte))) | (code << (8 * byte));
  }
  return word;
}

template <int LPG>
__device__ __forceinline__ uint32_t group_max_u32(uint32_t v) {
  // max over LPG adjacent lanes; every lane ends with the group's value
  if (LPG >= 2) v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  if (LPG >= 4) v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  if (LPG >= 8) v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x141, 0xF, 0xF, true));  // row_half_mirror
  if (LPG >= 16) v = max(v, (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x140, 0xF, 0xF, true)); // row_mirror
  if (LPG >= 32) v = max(v, (uint32_t)__shfl_xor((int)v, 16, 64));
  if (LPG >= 64) v = max(v, (uint32_t)__shfl_xor((int)v, 32, 64));
  return v;
}

// clamp of a value that is not NaN, in one instruction (the median of the three)
__device__ __forceinline__ float clamp_finite(float v, float lo, float hi) { return __builtin_amdgcn_fmed3f(v, lo, hi); }

// A lane's eight values (raw words as loaded) widened to fp32; returns the largest absolute bit pattern among them
// (NaN patterns compare above everything).
template <int XDT, int WORDS>
__device__ __forceinline__ uint32_t widen_chunk(const uint32_t (&w)[WORDS], float (&xv)[8]) {
  using E = Elem<XDT>;
  uint32_t m = 0u;
  if constexpr (WORDS == 4) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t lo = w[i] & 0xFFFFu, hi = w[i] >> 16;
      m = max(m, max(lo & E::kAbs, hi & E::kAbs));
      xv[2 * i] = E::widen(lo);
      xv[2 * i + 1] = E::widen(hi);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      m = max(m, w[i] & E::kAbs);
      xv[i] = E::widen(w[i]);
    }
  }
  return m;
}

// Eight values of a group whose largest absolute bit pattern is m -> their eight codes (two words) and the group's
// scale (the return value).  Every lane of a wavefront must call it: the branches are decided per wavefront.
template <int XDT>
__device__ __forceinline__ float quantize_chunk(const float (&xv)[8], uint32_t m, const QuantArgs& a, uint32_t& w0,
                                                uint32_t& w1) {
  using E = Elem<XDT>;
  float amax = E::widen(m);
  const bool special = m >= E::kInf;  // Inf or NaN somewhere in the group
  if (!(amax != amax)) amax = fmaxf(amax, a.floor);
  const float s = derive_scale(amax, a);
  const float r = 1.0f / s;

  // Decided once per wavefront (uniform branches): almost every wavefront holds finite inputs under finite
  // non-zero scales only, where no quotient can be NaN and a plain clamp finishes the job.
  // (a scale so small that its reciprocal overflows makes 0 * inf = NaN under the reciprocal rule: not plain either)
  const bool plain = __builtin_amdgcn_ballot_w64(special || !(s > 0.0f) || !(s < __builtin_huge_valf()) ||
                                                 !(r < __builtin_huge_valf())) == 0;
  float y[8];
  if (plain) {
    if (a.quotient_rule == FG_QUOT_RECIP_MUL) {
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = clamp_finite(xv[i] * r, a.lo, a.hi);
    } else if (__builtin_amdgcn_ballot_w64(!short_division_ok(false, s)) == 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = clamp_finite(short_division(xv[i], s, r), a.lo, a.hi);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = clamp_finite(xv[i] / s, a.lo, a.hi);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = unclamped_overflow(xv[i], s, r, quantize_value(xv[i], s, r, a), a);
  }
  w0 = pack2<false>(y[0], y[1], 0u, a.e5m2);
  w0 = pack2<true>(y[2], y[3], w0, a.e5m2);
  w1 = pack2<false>(y[4], y[5], 0u, a.e5m2);
  w1 = pack2<true>(y[6], y[7], w1, a.e5m2);
  if (!plain) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      w0 = fix_nan_byte(w0, i, y[i], a.e5m2);
      w1 = fix_nan_byte(w1, i, y[4 + i], a.e5m2);
    }
  }
  return s;
}

}  // namespace
}  // namespace fg
