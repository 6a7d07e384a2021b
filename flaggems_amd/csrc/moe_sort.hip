// Routing table of an expert layer: the routed slots in ascending order of their (local) expert, ties in slot order,
// and the cumulative ends of the experts' segments -- what the grouped GEMM takes as `row_index` and `offs`.
//
// Stands in for the sorting half of the reference's moe_align_block_size (src/flag_gems/fused/moe_align_block_size.py:
// 405-519: histogram, cumulative sum, scatter of the token ids by expert), without its padding of every expert to a
// multiple of the GEMM's BLOCK_M: the grouped kernel here takes arbitrary segment ends.  expert_map follows the
// reference's convention (global expert -> local expert or -1, moe_align_block_size.py:817-818); slots whose expert
// is not local, or not an expert at all, sort behind the last segment.  The same kernel also writes the reference's
// padded table itself (fg_moe_align_block_size: runs that start at multiples of the block size, the padding value,
// the expert of every block, the padded length) for callers that keep the reference's format.
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

// block_m == 0: the plain table (sorted slots, cumulative ends in `offs`).  block_m > 0: the padded table of the
// reference's moe_align_block_size -- every expert's run starts at a multiple of block_m, `sorted` (sorted_cap entries)
// holds n_slots wherever no slot lies, block_ids (block_cap entries) the expert of every block of block_m entries or
// -1, and *post_pad the padded length; slots without an expert are left out.
template <int ID_BYTES, int MAP_BYTES>
__global__ __launch_bounds__(kSortThreads) void moe_sort_slots_kernel(const void* __restrict__ ids, int n_slots, int experts,
                                                                      const void* __restrict__ map, int64_t map_len,
                                                                      int32_t* __restrict__ sorted, int32_t* __restrict__ offs,
                                                                      int block_m, int sorted_cap, int32_t* __restrict__ block_ids,
                                                                      int block_cap, int32_t* __restrict__ post_pad) {
  extern __shared__ int lds[];  // group sizes [kSortWaves][experts + 1], running bases [experts + 1]
  const int K = experts + 1;
  int* const sizes = lds;
  int* const base = lds + kSortWaves * K;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  for (int i = tid; i < (kSortWaves + 1) * K; i += kSortThreads) lds[i] = 0;
  if (block_m > 0) {
    for (int i = tid; i < sorted_cap; i += kSortThreads) sorted[i] = n_slots;
    for (int i = tid; i < block_cap; i += kSortThreads) block_ids[i] = -1;
  }
  __syncthreads();  // (also completes the fills above before any later store to the same entries)
  for (int s = tid; s < n_slots; s += kSortThreads) atomicAdd(&base[slot_key<ID_BYTES, MAP_BYTES>(ids, map, map_len, experts, s)], 1);
  __syncthreads();
  if (wave == 0) {  // exclusive scan of the counts, 64 keys at a time; the inclusive sums of the experts are `offs`
    int carry = 0;
    for (int c = 0; c < K; c += 64) {
      const int k = c + lane;
      const int count = k < K ? base[k] : 0;
      // the padded table rounds every expert's run up to whole blocks and has no run for slots without an expert
      const int v = block_m > 0 ? (k < experts ? (count + block_m - 1) / block_m * block_m : 0) : count;
      int incl = v;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
      }
      if (k < K) base[k] = carry + incl - v;
      if (k < experts && offs != nullptr) offs[k] = carry + incl;
      if (block_m > 0 && k < experts)
        for (int b = (carry + incl - v) / block_m; b < (carry + incl) / block_m && b < block_cap; ++b) block_ids[b] = k;
      carry += __shfl(incl, 63, 64);
    }
    if (block_m > 0 && lane == 0) *post_pad = carry;
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
    if (valid && !(block_m > 0 && k == experts)) {
      int pos = base[k] + rank;
      for (int w = 0; w < wave; ++w) pos += sizes[w * K + k];
      if (block_m == 0 || pos < sorted_cap) sorted[pos] = s;
    }
    __syncthreads();
    for (int i = tid; i < K; i += kSortThreads) {  // the key's base moves past the slots just placed; sizes back to zero
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

namespace fg {
namespace {
int launch_moe_sort(const char* me, const void* topk_ids, int id_bytes, int64_t n_slots, int64_t num_experts, const void* expert_map,
                    int map_bytes, int64_t map_len, int32_t* sorted_slots, int32_t* offs, int64_t block_m, int64_t sorted_cap,
                    int32_t* block_ids, int64_t block_cap, int32_t* post_pad, void* stream) {
  if (n_slots < 0 || num_experts < 1) FG_FAIL(FG_ERR_INVALID_ARG, "%s: %lld slots, %lld experts", me, (long long)n_slots, (long long)num_experts);
  if (num_experts > kSortMaxExperts || n_slots > kSortMaxSlots)
    FG_FAIL(FG_ERR_UNSUPPORTED, "%s: at most %d experts and %lld slots (got %lld, %lld)", me, kSortMaxExperts,
            (long long)kSortMaxSlots, (long long)num_experts, (long long)n_slots);
  if (n_slots > 0 && (!topk_ids || !sorted_slots)) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null pointer", me);
  if ((id_bytes != 4 && id_bytes != 8) || (expert_map != nullptr && map_bytes != 4 && map_bytes != 8))
    FG_FAIL(FG_ERR_INVALID_ARG, "%s: ids and map entries must be 4 or 8 bytes wide", me);
  if (expert_map != nullptr && map_len < 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: map length %lld", me, (long long)map_len);
  const int mb = expert_map ? map_bytes : 0;
  const size_t lds_bytes = (size_t)(kSortWaves + 1) * (size_t)(num_experts + 1) * sizeof(int);
  const dim3 grid(1), block(kSortThreads);
  hipStream_t st = (hipStream_t)stream;
  const int n = (int)n_slots, e = (int)num_experts, bm = (int)block_m, sc = (int)sorted_cap, bc = (int)block_cap;
#define FG_SORT_CASE(IB, MB) \
  if (id_bytes == IB && mb == MB) FG_LAUNCH((moe_sort_slots_kernel<IB, MB>), grid, block, lds_bytes, st, topk_ids, n, e, expert_map, map_len, sorted_slots, offs, bm, sc, block_ids, bc, post_pad)
  FG_SORT_CASE(8, 0); FG_SORT_CASE(8, 8); FG_SORT_CASE(8, 4);
  FG_SORT_CASE(4, 0); FG_SORT_CASE(4, 8); FG_SORT_CASE(4, 4);
#undef FG_SORT_CASE
  FG_CHECK_LAUNCH("moe_sort_slots_kernel");
  return FG_OK;
}
}  // namespace
}  // namespace fg

extern "C" int fg_moe_sort_slots(const void* topk_ids, int id_bytes, int64_t n_slots, int64_t num_experts, const void* expert_map,
                                 int map_bytes, int64_t map_len, int32_t* sorted_slots, int32_t* offs, void* stream) {
  if (!offs) FG_FAIL(FG_ERR_INVALID_ARG, "fg_moe_sort_slots: null pointer");
  return fg::launch_moe_sort("fg_moe_sort_slots", topk_ids, id_bytes, n_slots, num_experts, expert_map, map_bytes, map_len, sorted_slots,
                             offs, 0, 0, nullptr, 0, nullptr, stream);
}

extern "C" int fg_moe_align_block_size(const void* topk_ids, int id_bytes, int64_t n_slots, int64_t num_experts, int64_t block_size,
                                       int32_t* sorted_ids, int64_t sorted_cap, int32_t* expert_ids, int64_t expert_ids_cap,
                                       int32_t* num_tokens_post_pad, void* stream) {
  using namespace fg;
  const char* me = "fg_moe_align_block_size";
  if (block_size < 1 || block_size > 65536) FG_FAIL(FG_ERR_INVALID_ARG, "%s: block size %lld", me, (long long)block_size);
  if ((!sorted_ids && sorted_cap > 0) || (!expert_ids && expert_ids_cap > 0) || !num_tokens_post_pad) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null pointer", me);
  if (num_experts >= 1 && num_experts <= kSortMaxExperts && n_slots >= 0) {
    // the largest padded length: every expert's run rounded up
    const int64_t need = n_slots + num_experts * (block_size - 1);
    if (sorted_cap < need || sorted_cap > 0x7FFFFFFF || expert_ids_cap < (need + block_size - 1) / block_size || expert_ids_cap > 0x7FFFFFFF)
      FG_FAIL(FG_ERR_INVALID_ARG, "%s: %lld sorted entries and %lld block entries given, %lld and %lld needed", me, (long long)sorted_cap,
              (long long)expert_ids_cap, (long long)need, (long long)((need + block_size - 1) / block_size));
  }
  return launch_moe_sort(me, topk_ids, id_bytes, n_slots, num_experts, nullptr, 0, 0, sorted_ids, nullptr, block_size, sorted_cap,
                         expert_ids, expert_ids_cap, num_tokens_post_pad, stream);
}
