// Inverse rotary embedding fused into the FP8 group quantizer, the producer of the activations of DeepSeek-V4's grouped
// output projection (the "bhr,hdr->bhd" einsum):
//     o [tokens, heads, head_dim]  ->  q [groups, tokens, heads_per_group * head_dim] e4m3fn,  one scale per 128 values.
// The last rope_dim values of every head are rotated back by the token's position -- interleaved pairs,
//     even' = even * cos + odd * sin,     odd' = odd * cos - even * sin,     cos/sin = cache[position][i / 2], [half + i / 2]
// in fp32, without rounding to o's type -- and every group of `group_size` values is then quantized as
// fg_group_quant_fp8 quantizes it: amax floored at eps, scale = amax * fp32(1 / 448), optionally rounded up to a power of
// two, codes = clamp(x / scale) rounded to nearest even.  This follows the reference's kernel line by line
// (src/flag_gems/fused/fused_inv_rope_fp8_quant.py:38-161: rotation :96-113, scales :115-119, codes :128, packed
// exponents :139-149, padding rows :66-89).
//
// A wavefront takes one head of one token per step: 64 lanes x 8 values cover a head of 512 (longer heads take further
// passes), a rotated pair lies inside a lane, a 128-value group is 16 adjacent lanes (DPP maximum), and the eight lanes
// that hold the rope tail fetch their cos/sin once per token.  A wavefront walks HPW consecutive heads of a token with
// all loads issued first, then the next of its tokens.  HBM bound: 3 bytes per bf16 value.

#include "fp8_quant_device.h"

namespace fg {
namespace {

constexpr int kRopeThreads = 256;
constexpr int kRopeWaves = kRopeThreads / 64;

struct InvRopeArgs {
  const void* o;
  const void* positions;
  const float* cache;
  uint8_t* q;
  void* s;
  int64_t o_stride_token, o_stride_head, cache_stride;
  int64_t q_stride_group, q_stride_token;
  int64_t s_stride_group, s_stride_k;
  int tokens, heads, heads_per_group, head_dim, rope_start, half_rope, chunks_per_head, group_size;
  int pos_bytes, cache_rows, packed;
  QuantArgs qa;
};

__device__ __forceinline__ void rotate_back(float (&xv)[8], const float (&c)[4], const float (&s)[4]) {
  // products and sums rounded one by one, as the torch formula of the reference's test rounds them
#pragma clang fp contract(off)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float e = xv[2 * i], d = xv[2 * i + 1];
    xv[2 * i] = e * c[i] + d * s[i];
    xv[2 * i + 1] = d * c[i] - e * s[i];
  }
}

// Scales of one token are chunks * heads words scattered over as many columns (tokens have unit stride): a workgroup
// therefore takes kRopeTokens (16, or 4 in small launches) consecutive tokens of the same HPW heads, collects their scales in LDS and writes every
// column's words of those tokens as one run.
constexpr int kRopeLdsChunks = 16;  // groups per head that the LDS rows hold; longer heads store their scales directly

template <int XDT, int LPG, int HPW, int kRopeTokens, bool PACKED>
__global__ __launch_bounds__(kRopeThreads) void inv_rope_quant_kernel(InvRopeArgs a, int padded_tokens, int head_blocks) {
  // the rules are fixed for this producer: as constants they leave no rule switch in the loop
  a.qa.scale_rule = FG_SCALE_MUL_INV;
  a.qa.quotient_rule = FG_QUOT_DIV;
  a.qa.pow2_rule = PACKED ? FG_POW2_LOG2 : FG_POW2_NONE;
  a.qa.e5m2 = 0;
  a.packed = PACKED;
  constexpr int WORDS = XDT == FG_F32 ? 8 : 4;
  __shared__ uint32_t rows[HPW * kRopeLdsChunks][kRopeTokens];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // consecutive workgroups take the heads of the same tokens: together they read one contiguous stretch of o
  const int token_block = (int)(blockIdx.x / (uint32_t)head_blocks);
  const int64_t t0 = (int64_t)token_block * kRopeTokens;
  const int h_first = (int)(blockIdx.x - (uint32_t)token_block * (uint32_t)head_blocks) * HPW;
  const bool via_lds = a.chunks_per_head <= kRopeLdsChunks;
  const int words_per_head = a.packed ? 1 : a.chunks_per_head;

  // rows that pad the scale columns to a multiple of four tokens read as zero: whatever is not written below stays 0
  for (int i = threadIdx.x; i < HPW * kRopeLdsChunks * kRopeTokens; i += kRopeThreads) (&rows[0][0])[i] = 0u;
  __syncthreads();

  for (int tl = wave; tl < kRopeTokens; tl += kRopeWaves) {
    const int64_t t = t0 + tl;
    if (t >= a.tokens) break;  // uniform over the wavefront
    int64_t pos = a.pos_bytes == 8 ? reinterpret_cast<const int64_t*>(a.positions)[t]
                                   : (int64_t)reinterpret_cast<const int32_t*>(a.positions)[t];
    // the reference reads whatever lies at an out-of-range position; here the access stays inside the cache
    pos = pos < 0 ? 0 : (pos >= a.cache_rows ? a.cache_rows - 1 : pos);
    const float* const cs = a.cache + pos * a.cache_stride;

    for (int p0 = 0; p0 < a.head_dim; p0 += 512) {
      const int off = p0 + lane * 8;
      const bool live = off < a.head_dim;
      const bool rope = live && off >= a.rope_start;
      float cosv[4], sinv[4];
      if (rope) {
        const int idx = (off - a.rope_start) >> 1;
#pragma unroll
        for (int i = 0; i < 4; ++i) { cosv[i] = cs[idx + i]; sinv[i] = cs[a.half_rope + idx + i]; }
      }

      uint32_t w[HPW][WORDS];
#pragma unroll
      for (int i = 0; i < HPW; ++i) {
        const int h = h_first + i;
        const bool have = live && h < a.heads;
        const char* src = reinterpret_cast<const char*>(a.o) +
                          (t * a.o_stride_token + (int64_t)(have ? h : h_first) * a.o_stride_head + (live ? off : 0)) * (XDT == FG_F32 ? 4 : 2);
        const u32x4 v0 = *reinterpret_cast<const u32x4*>(src);
#pragma unroll
        for (int j = 0; j < 4; ++j) w[i][j] = have ? v0[j] : 0u;
        if constexpr (WORDS == 8) {
          const u32x4 v1 = *reinterpret_cast<const u32x4*>(src + 16);
#pragma unroll
          for (int j = 0; j < 4; ++j) w[i][4 + j] = have ? v1[j] : 0u;
        }
      }

#pragma unroll
      for (int i = 0; i < HPW; ++i) {
        const int h = h_first + i;
        if (h >= a.heads) break;  // uniform over the wavefront
        float xv[8];
        widen_chunk<XDT, WORDS>(w[i], xv);
        if (rope) rotate_back(xv, cosv, sinv);
        uint32_t m = 0u;
#pragma unroll
        for (int j = 0; j < 8; ++j) m = max(m, float_to_bits(xv[j]) & 0x7FFFFFFFu);
        m = group_max_u32<LPG>(m);
        uint32_t w0, w1;
        const float s = quantize_chunk<FG_F32>(xv, m, a.qa, w0, w1);

        const int g = h / a.heads_per_group, hig = h - g * a.heads_per_group;
        if (live) {
          uint8_t* dst = a.q + g * a.q_stride_group + t * a.q_stride_token + (int64_t)hig * a.head_dim + off;
          *reinterpret_cast<uint2*>(dst) = make_uint2(w0, w1);
        }
        if (a.packed) {
          // one word per head: byte c is the exponent field of group c's scale (a power of two)
          const uint32_t e = (float_to_bits(s) >> 23) & 0xFFu;
          uint32_t word = 0u;
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const uint32_t ec = (uint32_t)__builtin_amdgcn_readlane((int)e, (c * LPG) & 63);
            if (c < a.chunks_per_head) word |= ec << (8 * c);
          }
          if (lane == 0) rows[i][tl] = word;
        } else if (live && (lane & (LPG - 1)) == 0) {
          const int chunk = off / a.group_size;
          if (via_lds) rows[i * a.chunks_per_head + chunk][tl] = float_to_bits(s);
          else reinterpret_cast<float*>(a.s)[g * a.s_stride_group + t + (int64_t)(hig * a.chunks_per_head + chunk) * a.s_stride_k] = s;
        }
      }
    }
  }
  __syncthreads();

  // column by column: kRopeTokens consecutive words each
  if (via_lds) {
    for (int i = threadIdx.x; i < HPW * words_per_head * kRopeTokens; i += kRopeThreads) {
      const int row = i / kRopeTokens, tl = i - row * kRopeTokens;
      const int hl = row / words_per_head, c = row - hl * words_per_head;
      const int h = h_first + hl;
      const int64_t t = t0 + tl;
      if (h >= a.heads || t >= padded_tokens) continue;
      const int g = h / a.heads_per_group, hig = h - g * a.heads_per_group;
      reinterpret_cast<uint32_t*>(a.s)[g * a.s_stride_group + t + (int64_t)(hig * words_per_head + c) * a.s_stride_k] = rows[row][tl];
    }
  } else {
    // heads too long for the LDS rows: only the padding rows are left to write
    for (int i = threadIdx.x; i < HPW * words_per_head * kRopeTokens; i += kRopeThreads) {
      const int row = i / kRopeTokens, tl = i - row * kRopeTokens;
      const int hl = row / words_per_head, c = row - hl * words_per_head;
      const int h = h_first + hl;
      const int64_t t = t0 + tl;
      if (h >= a.heads || t < a.tokens || t >= padded_tokens) continue;
      const int g = h / a.heads_per_group, hig = h - g * a.heads_per_group;
      reinterpret_cast<uint32_t*>(a.s)[g * a.s_stride_group + t + (int64_t)(hig * words_per_head + c) * a.s_stride_k] = 0u;
    }
  }
}

template <int XDT, int LPG>
int launch_inv_rope(const InvRopeArgs& a, int64_t padded_tokens, hipStream_t stream) {
  // 16 tokens and four heads per workgroup once that leaves workgroups enough to fill the GPU; else 4 tokens, one head
  const bool wide = ceil_div(padded_tokens, (int64_t)16) * (a.heads / 4) >= 1024 && a.heads % 4 == 0;
  const int64_t head_blocks = wide ? a.heads / 4 : a.heads;
  const int64_t blocks = ceil_div(padded_tokens, (int64_t)(wide ? 16 : 4)) * head_blocks;
  if (blocks > 0x7FFFFFFF) FG_FAIL(FG_ERR_UNSUPPORTED, "fg_inv_rope_group_quant_fp8: too many workgroups");
  const dim3 grid((uint32_t)blocks);
  if (wide && a.packed) FG_LAUNCH((inv_rope_quant_kernel<XDT, LPG, 4, 16, true>), grid, dim3(kRopeThreads), 0, stream, a, (int)padded_tokens, (int)head_blocks);
  else if (wide) FG_LAUNCH((inv_rope_quant_kernel<XDT, LPG, 4, 16, false>), grid, dim3(kRopeThreads), 0, stream, a, (int)padded_tokens, (int)head_blocks);
  else if (a.packed) FG_LAUNCH((inv_rope_quant_kernel<XDT, LPG, 1, 4, true>), grid, dim3(kRopeThreads), 0, stream, a, (int)padded_tokens, (int)head_blocks);
  else FG_LAUNCH((inv_rope_quant_kernel<XDT, LPG, 1, 4, false>), grid, dim3(kRopeThreads), 0, stream, a, (int)padded_tokens, (int)head_blocks);
  return FG_OK;
}

template <int XDT>
int launch_inv_rope_group(const InvRopeArgs& a, int64_t padded_tokens, hipStream_t stream) {
  switch (a.group_size) {
    case 64: if (int rc = launch_inv_rope<XDT, 8>(a, padded_tokens, stream)) return rc; break;
    case 128: if (int rc = launch_inv_rope<XDT, 16>(a, padded_tokens, stream)) return rc; break;
    case 256: if (int rc = launch_inv_rope<XDT, 32>(a, padded_tokens, stream)) return rc; break;
    case 512: if (int rc = launch_inv_rope<XDT, 64>(a, padded_tokens, stream)) return rc; break;
    default: FG_FAIL(FG_ERR_UNSUPPORTED, "fg_inv_rope_group_quant_fp8: group size %d (64, 128, 256 or 512)", a.group_size);
  }
  FG_CHECK_LAUNCH("inv_rope_quant_kernel");
  return FG_OK;
}

}  // namespace
}  // namespace fg

extern "C" int fg_inv_rope_group_quant_fp8(const void* o, int o_dtype, int64_t tokens, int64_t heads, int64_t head_dim,
                                           int64_t o_stride_token, int64_t o_stride_head,
                                           const void* positions, int position_bytes,
                                           const float* cos_sin_cache, int64_t cache_rows, int64_t cache_stride,
                                           int64_t heads_per_group, int64_t rope_dim, int64_t group_size, float eps,
                                           void* q, int64_t q_stride_group, int64_t q_stride_token,
                                           void* scales, int64_t scale_stride_group, int64_t scale_stride_k,
                                           int64_t padded_tokens, int pack_ue8m0, void* stream) {
  using namespace fg;
  const char* me = "fg_inv_rope_group_quant_fp8";
  if (tokens < 0 || heads < 0 || head_dim < 0 || padded_tokens < tokens) FG_FAIL(FG_ERR_INVALID_ARG, "%s: negative size", me);
  if (padded_tokens == 0 || heads == 0 || head_dim == 0) return FG_OK;
  if (!o || !positions || !cos_sin_cache || !q || !scales) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null pointer", me);
  if (o_dtype != FG_BF16 && o_dtype != FG_F16 && o_dtype != FG_F32) FG_FAIL(FG_ERR_INVALID_ARG, "%s: o_dtype %d", me, o_dtype);
  if (position_bytes != 4 && position_bytes != 8) FG_FAIL(FG_ERR_INVALID_ARG, "%s: positions of %d bytes", me, position_bytes);
  if (heads_per_group < 1 || heads % heads_per_group != 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: %lld heads in groups of %lld", me, (long long)heads, (long long)heads_per_group);
  if (group_size < 1 || head_dim % group_size != 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: head_dim %lld is not a multiple of the group size %lld", me, (long long)head_dim, (long long)group_size);
  if (rope_dim < 0 || rope_dim > group_size || rope_dim > head_dim || rope_dim % 2 != 0)
    FG_FAIL(FG_ERR_INVALID_ARG, "%s: rope_dim %lld must be even and lie inside the last group", me, (long long)rope_dim);
  if (cache_rows < 1 || cache_stride < rope_dim) FG_FAIL(FG_ERR_INVALID_ARG, "%s: cos/sin cache of %lld rows, stride %lld", me, (long long)cache_rows, (long long)cache_stride);
  if (rope_dim % 8 != 0) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: rope_dim %lld is not a multiple of 8", me, (long long)rope_dim);
  if (padded_tokens > 0x7FFFFFFF || heads > (1 << 20) || head_dim > (1 << 20) || cache_rows > 0x7FFFFFFF)
    FG_FAIL(FG_ERR_UNSUPPORTED, "%s: dimension too large", me);
  const int64_t chunks = head_dim / group_size;
  if (pack_ue8m0 && (chunks > 4 || head_dim > 512)) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: packed exponents take at most four groups per head", me);
  const int64_t esz = o_dtype == FG_F32 ? 4 : 2;
  if ((uintptr_t)o % 16 != 0 || (o_stride_token * esz) % 16 != 0 || (o_stride_head * esz) % 16 != 0 || (uintptr_t)q % 8 != 0 ||
      q_stride_group % 8 != 0 || q_stride_token % 8 != 0)
    FG_FAIL(FG_ERR_UNSUPPORTED, "%s: heads of o must be 16-byte aligned and rows of q 8-byte aligned", me);

  InvRopeArgs a = {};
  a.o = o; a.positions = positions; a.cache = cos_sin_cache;
  a.q = reinterpret_cast<uint8_t*>(q); a.s = scales;
  a.o_stride_token = o_stride_token; a.o_stride_head = o_stride_head; a.cache_stride = cache_stride;
  a.q_stride_group = q_stride_group; a.q_stride_token = q_stride_token;
  a.s_stride_group = scale_stride_group; a.s_stride_k = scale_stride_k;
  a.tokens = (int)tokens; a.heads = (int)heads; a.heads_per_group = (int)heads_per_group; a.head_dim = (int)head_dim;
  a.rope_start = (int)(head_dim - rope_dim); a.half_rope = (int)(rope_dim / 2);
  a.chunks_per_head = (int)chunks; a.group_size = (int)group_size;
  a.pos_bytes = position_bytes; a.cache_rows = (int)cache_rows; a.packed = pack_ue8m0 != 0;
  a.qa.floor = eps; a.qa.lo = -448.0f; a.qa.hi = 448.0f; a.qa.inv_max = 1.0f / 448.0f;
  a.qa.scale_rule = FG_SCALE_MUL_INV; a.qa.quotient_rule = FG_QUOT_DIV;
  a.qa.pow2_rule = pack_ue8m0 ? FG_POW2_LOG2 : FG_POW2_NONE; a.qa.e5m2 = 0;
  if (o_dtype == FG_BF16) return launch_inv_rope_group<FG_BF16>(a, padded_tokens, (hipStream_t)stream);
  if (o_dtype == FG_F16) return launch_inv_rope_group<FG_F16>(a, padded_tokens, (hipStream_t)stream);
  return launch_inv_rope_group<FG_F32>(a, padded_tokens, (hipStream_t)stream);
}
