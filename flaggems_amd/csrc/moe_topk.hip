// Routing of an expert layer, the step before fused_experts_impl: which experts a token goes to and with what weight.
//
//   fg_topk_softmax   softmax over the experts, the k largest probabilities in descending order (ties: the lower
//                     expert first), optionally renormalised to sum 1
//                     (src/flag_gems/fused/topk_softmax.py:24-82: exp(x - max) / (sum + 1e-8), k rounds of max / argmax,
//                     value / (sum of the selected + 1e-8)).
//   fg_grouped_topk   DeepSeek's group-limited routing: a group's score is the sum of its two largest biased
//                     scores, the topk_group best groups stay, the k best biased scores among their experts are
//                     selected, and the weights are the unbiased scores times routed_scaling_factor, optionally over
//                     their sum (src/flag_gems/fused/grouped_topk.py:25-78 group scores, :81-253 selection).
//
// Both are a few hundred bytes per token and bound by latency, not by any roofline: one wavefront per token, the
// experts dealt to the lanes (expert e in lane e % 64, slot e / 64), every maximum a 64-bit key (order-preserving
// image of the value above the complement of the index, so that the largest key is the largest value at the lowest
// index) reduced over the wavefront with six exchanges, four of them DPP moves inside a row of 16 lanes.

#include "fg_common.h"

namespace fg {
namespace {

constexpr int kTopkThreads = 256;
constexpr int kTopkWaves = kTopkThreads / 64;

__device__ __forceinline__ float load_elem(const void* p, int64_t i, int dt) {
  if (dt == FG_F32) return reinterpret_cast<const float*>(p)[i];
  if (dt == FG_F16) return (float)reinterpret_cast<const _Float16*>(p)[i];
  return bits_to_float((uint32_t)reinterpret_cast<const uint16_t*>(p)[i] << 16);
}
// round to the tensor's type and back (what an operation on 16-bit tensors keeps)
__device__ __forceinline__ float round_like(float v, int dt) {
  if (dt == FG_F32) return v;
  if (dt == FG_F16) return (float)(_Float16)v;
  const uint32_t u = float_to_bits(v);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return v;
  return bits_to_float((u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u);
}
// order-preserving image of a float in an unsigned word (-inf lowest, +inf highest; NaN is not ordered)
__device__ __forceinline__ uint32_t ordered(float v) {
  const uint32_t u = float_to_bits(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float unordered(uint32_t o) { return bits_to_float((o & 0x80000000u) ? (o & 0x7FFFFFFFu) : ~o); }
__device__ __forceinline__ uint64_t make_key(float v, uint32_t index) { return ((uint64_t)ordered(v) << 32) | (uint64_t)(~index); }

// A value of another lane: the four exchanges inside a row of 16 lanes are DPP moves (quad swaps, then mirrors of 8 and
// of 16 lanes: for a reduction any pairing across the halves serves), the two across rows go through the LDS crossbar.
template <int STEP>
__device__ __forceinline__ uint32_t from_partner(uint32_t v) {
  if (STEP == 0) return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);   // quad_perm [1, 0, 3, 2]
  if (STEP == 1) return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true);   // quad_perm [2, 3, 0, 1]
  if (STEP == 2) return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x141, 0xF, 0xF, true);  // row_half_mirror
  if (STEP == 3) return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x140, 0xF, 0xF, true);  // row_mirror
  return (uint32_t)__shfl_xor((int)v, STEP == 4 ? 16 : 32, 64);
}
template <int STEP>
__device__ __forceinline__ float from_partner_f32(float v) { return bits_to_float(from_partner<STEP>(float_to_bits(v))); }

template <int STEP = 0>
__device__ __forceinline__ uint64_t wave_max_key(uint64_t k) {
  const uint64_t o = ((uint64_t)from_partner<STEP>((uint32_t)(k >> 32)) << 32) | from_partner<STEP>((uint32_t)k);
  k = o > k ? o : k;
  if constexpr (STEP < 5) return wave_max_key<STEP + 1>(k);
  return k;
}
template <int STEP = 0>
__device__ __forceinline__ float wave_max_f32(float v) {
  v = fmaxf(v, from_partner_f32<STEP>(v));
  if constexpr (STEP < 5) return wave_max_f32<STEP + 1>(v);
  return v;
}
// (largest, second largest) over the wavefront of the lanes' (t1, t2) pairs
template <int STEP = 0>
__device__ __forceinline__ void wave_top2_f32(float& t1, float& t2) {
  const float o1 = from_partner_f32<STEP>(t1), o2 = from_partner_f32<STEP>(t2);
  t2 = fmaxf(fminf(t1, o1), fmaxf(t2, o2));
  t1 = fmaxf(t1, o1);
  if constexpr (STEP < 5) wave_top2_f32<STEP + 1>(t1, t2);
}
__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) v = v + __shfl_xor(v, d, 64);
  return v;
}

template <int VPL>
__global__ __launch_bounds__(kTopkThreads) void topk_softmax_kernel(const void* __restrict__ gating, int dt, int64_t row_stride,
                                                                    int tokens, int experts, int k, int renormalize,
                                                                    float* __restrict__ weights, void* __restrict__ indices,
                                                                    int index_bytes, int* __restrict__ token_expert) {
  const int lane = threadIdx.x & 63;
  const int row = (int)blockIdx.x * kTopkWaves + (int)(threadIdx.x >> 6);
  if (row >= tokens) return;  // the whole wavefront
  float x[VPL];
  float m = -__builtin_huge_valf();
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = lane + 64 * i;
    x[i] = e < experts ? load_elem(gating, (int64_t)row * row_stride + e, dt) : -__builtin_huge_valf();
    m = fmaxf(m, x[i]);
  }
  m = wave_max_f32(m);
  float part = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    x[i] = (lane + 64 * i) < experts ? expf(x[i] - m) : 0.f;
    part = part + x[i];
  }
  const float denom = wave_sum_f32(part) + 1e-8f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) x[i] = x[i] / denom;

  float my_val = 0.f, selected_sum = 0.f;
  uint32_t my_idx = 0u;
  for (int ki = 0; ki < k; ++ki) {
    uint64_t best = 0;  // below every key of a valid expert
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const uint32_t e = (uint32_t)(lane + 64 * i);
      const uint64_t key = (int)e < experts ? make_key(x[i], e) : 0ull;
      best = key > best ? key : best;
    }
    best = wave_max_key(best);
    const uint32_t e = ~(uint32_t)best;
    const float v = unordered((uint32_t)(best >> 32));
    selected_sum = selected_sum + v;
    if (lane == ki) { my_val = v; my_idx = e; }
#pragma unroll
    for (int i = 0; i < VPL; ++i)
      if ((uint32_t)(lane + 64 * i) == e) x[i] = -__builtin_huge_valf();  // taken: below every probability
  }
  if (lane < k) {
    const int64_t o = (int64_t)row * k + lane;
    weights[o] = renormalize ? my_val / (selected_sum + 1e-8f) : my_val;
    if (index_bytes == 8) reinterpret_cast<int64_t*>(indices)[o] = (int64_t)my_idx;
    else reinterpret_cast<uint32_t*>(indices)[o] = my_idx;
    if (token_expert != nullptr) token_expert[o] = lane * tokens + row;
  }
}

struct GroupedTopkArgs {
  const void* scores;
  const void* bias;
  float* values;
  int* ids;
  int64_t score_stride, out_stride;
  int dt, tokens, experts, n_group, topk_group, topk, per_group, renormalize, sigmoid;
  float scaling;
};

template <int VPL>
__global__ __launch_bounds__(kTopkThreads) void grouped_topk_kernel(GroupedTopkArgs a) {
  const int lane = threadIdx.x & 63;
  const int row = (int)blockIdx.x * kTopkWaves + (int)(threadIdx.x >> 6);
  if (row >= a.tokens) return;  // the whole wavefront
  const float kNegInf = -__builtin_huge_valf();
  float s[VPL], sb[VPL];  // the score (after the scoring function, in the tensor's type) and score + bias
  int grp[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = lane + 64 * i;
    const bool in = e < a.experts;
    float v = in ? load_elem(a.scores, (int64_t)row * a.score_stride + e, a.dt) : kNegInf;
    if (a.sigmoid && in) v = round_like(1.0f / (1.0f + expf(-v)), a.dt);
    s[i] = v;
    sb[i] = in ? round_like(v + load_elem(a.bias, e, a.dt), a.dt) : kNegInf;
    grp[i] = in ? e / a.per_group : -1;
  }

  // group scores: the two largest biased scores of a group (the largest twice when it occurs twice), lane g holds group g's
  float group_score = kNegInf;
  for (int g = 0; g < a.n_group; ++g) {
    // (largest, second largest) of the lane's values, then of pairs of lanes: no index is needed here
    float t1 = kNegInf, t2 = kNegInf;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const float v = grp[i] == g ? sb[i] : kNegInf;
      t2 = fmaxf(t2, fminf(t1, v));
      t1 = fmaxf(t1, v);
    }
    wave_top2_f32(t1, t2);
    // (a group of one expert has no second score: -inf, as the reference's maximum over nothing)
    const float gs = round_like(t1 + t2, a.dt);
    if (lane == g) group_score = gs;
  }
  // scores that are not finite count as -inf; no group above -inf: the reference's fixed answer
  if (!(group_score == group_score) || group_score == __builtin_huge_valf()) group_score = kNegInf;
  const bool proceed = wave_max_f32(lane < a.n_group ? group_score : kNegInf) != kNegInf;

  // the topk_group best groups, ties to the lower group
  uint32_t chosen = 0u;
  float gs_left = group_score;
  for (int r = 0; r < a.topk_group; ++r) {
    const uint64_t best = wave_max_key(lane < a.n_group && !((chosen >> lane) & 1u) ? make_key(gs_left, (uint32_t)lane) : 0ull);
    if (best == 0) break;
    chosen |= 1u << (~(uint32_t)best & 31u);
  }

  float sel[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) sel[i] = (grp[i] >= 0 && ((chosen >> grp[i]) & 1u)) ? sb[i] : kNegInf;

  float my_val = 0.f, total = 0.f;
  int my_idx = 0;
  for (int ki = 0; ki < a.topk; ++ki) {
    uint64_t best = 0;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const uint32_t e = (uint32_t)(lane + 64 * i);
      const uint64_t key = (int)e < a.experts ? make_key(sel[i], e) : 0ull;
      best = key > best ? key : best;
    }
    best = wave_max_key(best);
    const uint32_t e = ~(uint32_t)best;
    // the weight is the score without the bias
    float mine = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; ++i)
      if ((uint32_t)i == (e >> 6)) mine = s[i];
    const float v = __shfl(mine, (int)(e & 63u), 64);
    total = total + v;
    if (lane == ki) { my_val = v; my_idx = (int)e; }
#pragma unroll
    for (int i = 0; i < VPL; ++i)
      if ((uint32_t)(lane + 64 * i) == e) sel[i] = kNegInf;
  }
  if (lane < a.topk) {
    const float scale = a.renormalize ? a.scaling / (total + 1e-20f) : a.scaling;
    const int64_t o = (int64_t)row * a.out_stride + lane;
    a.values[o] = proceed ? my_val * scale : 1.0f / (float)a.topk;
    a.ids[o] = proceed ? my_idx : lane;
  }
}

}  // namespace
}  // namespace fg

extern "C" int fg_topk_softmax(const void* gating, int dtype, int64_t tokens, int64_t experts, int64_t row_stride,
                               int64_t topk, int renormalize, float* topk_weights, void* topk_indices, int index_bytes,
                               int* token_expert_indices, void* stream) {
  using namespace fg;
  const char* me = "fg_topk_softmax";
  if (tokens < 0 || experts < 0 || topk < 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: negative size", me);
  if (tokens == 0 || topk == 0) return FG_OK;
  if (!gating || !topk_weights || !topk_indices) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null pointer", me);
  if (dtype != FG_BF16 && dtype != FG_F16 && dtype != FG_F32) FG_FAIL(FG_ERR_INVALID_ARG, "%s: dtype %d", me, dtype);
  if (index_bytes != 4 && index_bytes != 8) FG_FAIL(FG_ERR_INVALID_ARG, "%s: indices of %d bytes", me, index_bytes);
  if (topk > 32 || topk > experts) FG_FAIL(FG_ERR_INVALID_ARG, "%s: topk %lld of %lld experts (at most 32)", me, (long long)topk, (long long)experts);
  if (experts > 1024) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: more than 1024 experts", me);
  if (row_stride < experts || tokens > 0x7FFFFFFF / 32) FG_FAIL(FG_ERR_INVALID_ARG, "%s: row stride or token count", me);
  const dim3 grid((uint32_t)ceil_div(tokens, (int64_t)kTopkWaves)), block(kTopkThreads);
  const int T = (int)tokens, E = (int)experts, K = (int)topk;
#define FG_TOPK_CASE(V) FG_LAUNCH(topk_softmax_kernel<V>, grid, block, 0, (hipStream_t)stream, gating, dtype, row_stride, T, E, K, renormalize, topk_weights, topk_indices, index_bytes, token_expert_indices)
  if (E <= 64) FG_TOPK_CASE(1);
  else if (E <= 128) FG_TOPK_CASE(2);
  else if (E <= 256) FG_TOPK_CASE(4);
  else if (E <= 512) FG_TOPK_CASE(8);
  else FG_TOPK_CASE(16);
#undef FG_TOPK_CASE
  FG_CHECK_LAUNCH("topk_softmax_kernel");
  return FG_OK;
}

extern "C" int fg_grouped_topk(const void* scores, int dtype, int64_t tokens, int64_t experts, int64_t score_stride,
                               const void* bias, int64_t n_group, int64_t topk_group, int64_t topk, int renormalize,
                               float routed_scaling_factor, int scoring_func, float* topk_values, int* topk_ids,
                               int64_t out_stride, void* stream) {
  using namespace fg;
  const char* me = "fg_grouped_topk";
  if (tokens < 0 || experts < 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: negative size", me);
  if (tokens == 0 || topk <= 0) return FG_OK;
  if (!scores || !bias || !topk_values || !topk_ids) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null pointer", me);
  if (dtype != FG_BF16 && dtype != FG_F16 && dtype != FG_F32) FG_FAIL(FG_ERR_INVALID_ARG, "%s: dtype %d", me, dtype);
  if (n_group < 1 || n_group > 32 || experts % n_group != 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: %lld experts in %lld groups (at most 32)", me, (long long)experts, (long long)n_group);
  if (topk > 32 || topk > experts || topk_group < 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: topk %lld, topk_group %lld", me, (long long)topk, (long long)topk_group);
  if (scoring_func != 0 && scoring_func != 1) FG_FAIL(FG_ERR_INVALID_ARG, "%s: scoring_func %d", me, scoring_func);
  if (experts > 1024) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: more than 1024 experts", me);
  if (score_stride < experts || out_stride < topk || tokens > 0x7FFFFFFF / 32) FG_FAIL(FG_ERR_INVALID_ARG, "%s: strides or token count", me);
  GroupedTopkArgs a;
  a.scores = scores; a.bias = bias; a.values = topk_values; a.ids = topk_ids;
  a.score_stride = score_stride; a.out_stride = out_stride;
  a.dt = dtype; a.tokens = (int)tokens; a.experts = (int)experts; a.n_group = (int)n_group;
  a.topk_group = (int)(topk_group < n_group ? topk_group : n_group); a.topk = (int)topk; a.per_group = (int)(experts / n_group);
  a.renormalize = renormalize != 0; a.sigmoid = scoring_func == 1; a.scaling = routed_scaling_factor;
  const dim3 grid((uint32_t)ceil_div(tokens, (int64_t)kTopkWaves)), block(kTopkThreads);
  const int E = (int)experts;
  if (E <= 64) FG_LAUNCH(grouped_topk_kernel<1>, grid, block, 0, (hipStream_t)stream, a);
  else if (E <= 128) FG_LAUNCH(grouped_topk_kernel<2>, grid, block, 0, (hipStream_t)stream, a);
  else if (E <= 256) FG_LAUNCH(grouped_topk_kernel<4>, grid, block, 0, (hipStream_t)stream, a);
  else if (E <= 512) FG_LAUNCH(grouped_topk_kernel<8>, grid, block, 0, (hipStream_t)stream, a);
  else FG_LAUNCH(grouped_topk_kernel<16>, grid, block, 0, (hipStream_t)stream, a);
  FG_CHECK_LAUNCH("grouped_topk_kernel");
  return FG_OK;
}
