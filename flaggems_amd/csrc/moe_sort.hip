// Routing table of an expert layer: the routed slots in ascending order of their (local) expert, ties in slot order,
// and the cumulative ends of the experts' segments -- what the grouped GEMM takes as `row_index` and `offs`.
//
// Stands in for the sorting half of the reference's moe_align_block_size (src/flag_gems/fused/moe_align_block_size.py:
// 405-519: histogram, cumulative sum, scatter of the token ids by expert), without its padding of every expert to a
// multiple of the GEMM's BLOCK_M: the grouped kernel here takes arbitrary segment ends.  expert_map follows the
// reference's convention (global expert -> local expert or -1, moe_align_block_size.py:817-818); slots whose expert
// is not local, or not an expert at all, sort behind the last segment.
//
// One block of 16 wavefronts does the whole job (a table of at most 65536 slots is a few tens of KB: launch latency,
// not bandwidth, is what a second kernel would cost).  Pass 1 counts the keys with LDS atomics and scans the counts.
// Pass 2 walks the slots 1024 at a time, in order: inside a wavefront a lane finds the lanes with its key through
// ballots over the key's bits (its rank among them is a population count), the first lane of every such group
// records the group's size per wavefront and key, and after a barrier a slot's position is the key's running base
// plus the sizes recorded by the wavefronts before its own plus its rank: a stable counting sort whose output does
// not depend on timing.

#include "fg_common.h"

namespace fg {
namespace {

constexpr int kSortThreads = 1024;
constexpr int kSortWaves = kSortThreads / 64;
constexpr int kSortMaxExperts = 960;  // (16 + 1) tables of experts + 1 counters within the 64 KB of LDS a block gets without asking
constexpr int64_t kSortMaxSlots = 65536;

template <typename T>
__device__ __forceinline__ int64_t load_int(const void* p, int64_t i) { return (int64_t)reinterpret_cast<const T*>(p)[i]; }

// key of slot s: its local expert, or `experts` when it has none
template <int ID_BYTES, int MAP_BYTES>
__device__ __forceinline__ int slot_key(const void* ids, const void* map, int64_t map_len, int experts, int64_t s) {
  int64_t e = ID_BYTES == 8 ? load_int<int64_t>(ids, s) : load_int<int32_t>(ids, s);
  if (MAP_BYTES != 0) {
    if (e < 0 || e >= map_len) return experts;
    e = MAP_BYTES == 8 ? load_int<int64_t>(map, e) : load_int<int32_t>(map, e);
  }
  return (e >= 0 && e < experts) ? (int)e : experts;
}

template <int ID_BYTES, int MAP_BYTES>
__global__ __launch_bounds__(kSortThreads) void moe_sort_slots_kernel(const void* __restrict__ ids, int n_slots, int experts,
                                                                      const void* __restrict__ map, int64_t map_len,
                                                                      int32_t* __restrict__ sorted, int32_t* __restrict__ offs) {
  extern __shared__ int lds[];  // group sizes [kSortWaves][experts + 1], running bases [experts + 1]
  const int K = experts + 1;
  int* const sizes = lds;
  int* const base = lds + kSortWaves * K;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  for (int i = tid; i < (kSortWaves + 1) * K; i += kSortThreads) lds[i] = 0;
  __syncthreads();
  for (int s = tid; s < n_slots; s += kSortThreads) atomicAdd(&base[slot_key<ID_BYTES, MAP_BYTES>(ids, map, map_len, experts, s)], 1);
  __syncthreads();
  if (wave == 0) {  // exclusive scan of the counts, 64 keys at a time; the inclusive sums of the experts are `offs`
    int carry = 0;
    for (int c = 0; c < K; c += 64) {
      const int k = c + lane;
      const int v = k < K ? base[k] : 0;
      int incl = v;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
      }
      if (k < K) base[k] = carry + incl - v;
      if (k < experts) offs[k] = carry + incl;
      carry += __shfl(incl, 63, 64);
    }
  }
  __syncthreads();

  for (int c0 = 0; c0 < n_slots; c0 += kSortThreads) {
    const int s = c0 + tid;
    const bool valid = s < n_slots;
    const int k = valid ? slot_key<ID_BYTES, MAP_BYTES>(ids, map, map_len, experts, s) : 0;
    // lanes of this wavefront that hold a slot with the same key (keys are at most 960: 10 bits)
    uint64_t same = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 10; ++b) {
      const bool bit = (k >> b) & 1;
      const uint64_t with_bit = __ballot(bit);
      same &= bit ? with_bit : ~with_bit;
    }
    const int rank = __popcll(same & ((1ull << lane) - 1ull));
    if (valid && rank == 0) sizes[wave * K + k] = __popcll(same);
    __syncthreads();
    if (valid) {
      int pos = base[k] + rank;
      for (int w = 0; w < wave; ++w) pos += sizes[w * K + k];
      sorted[pos] = s;
    }
    __syncthreads();
    for (int i = tid; i < K; i += kSortThreads) {  // the key's base moves past this round's slots; sizes back to zero
      int t = 0;
#pragma unroll
      for (int w = 0; w < kSortWaves; ++w) {
        t += sizes[w * K + i];
        sizes[w * K + i] = 0;
      }
      base[i] += t;
    }
    __syncthreads();
  }
}

}  // namespace
}  // namespace fg

extern "C" int fg_moe_sort_slots(const void* topk_ids, int id_bytes, int64_t n_slots, int64_t num_experts, const void* expert_map,
                                 int map_bytes, int64_t map_len, int32_t* sorted_slots, int32_t* offs, void* stream) {
  using namespace fg;
  if (n_slots < 0 || num_experts < 1) FG_FAIL(FG_ERR_INVALID_ARG, "fg_moe_sort_slots: %lld slots, %lld experts", (long long)n_slots, (long long)num_experts);
  if (num_experts > kSortMaxExperts || n_slots > kSortMaxSlots)
    FG_FAIL(FG_ERR_UNSUPPORTED, "fg_moe_sort_slots: at most %d experts and %lld slots (got %lld, %lld)", kSortMaxExperts,
            (long long)kSortMaxSlots, (long long)num_experts, (long long)n_slots);
  if (!offs || (n_slots > 0 && (!topk_ids || !sorted_slots))) FG_FAIL(FG_ERR_INVALID_ARG, "fg_moe_sort_slots: null pointer");
  if ((id_bytes != 4 && id_bytes != 8) || (expert_map != nullptr && map_bytes != 4 && map_bytes != 8))
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_moe_sort_slots: ids and map entries must be 4 or 8 bytes wide");
  if (expert_map != nullptr && map_len < 0) FG_FAIL(FG_ERR_INVALID_ARG, "fg_moe_sort_slots: map length %lld", (long long)map_len);
  const int mb = expert_map ? map_bytes : 0;
  const size_t lds_bytes = (size_t)(kSortWaves + 1) * (size_t)(num_experts + 1) * sizeof(int);
  const dim3 grid(1), block(kSortThreads);
  hipStream_t st = (hipStream_t)stream;
  const int n = (int)n_slots, e = (int)num_experts;
#define FG_SORT_CASE(IB, MB) \
  if (id_bytes == IB && mb == MB) FG_LAUNCH((moe_sort_slots_kernel<IB, MB>), grid, block, lds_bytes, st, topk_ids, n, e, expert_map, map_len, sorted_slots, offs)
  FG_SORT_CASE(8, 0); FG_SORT_CASE(8, 8); FG_SORT_CASE(8, 4);
  FG_SORT_CASE(4, 0); FG_SORT_CASE(4, 8); FG_SORT_CASE(4, 4);
#undef FG_SORT_CASE
  FG_CHECK_LAUNCH("moe_sort_slots_kernel");
  return FG_OK;
}
