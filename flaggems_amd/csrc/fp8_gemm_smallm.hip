// Small-M (decode) FP8 GEMM for gfx950: M <= 64 activation rows against an [N, K] weight that is read
// exactly once.  The kernels are bound by HBM bandwidth and, for launches of a few microseconds, by what a
// compute unit does before and after its bytes arrive, so the design is about bytes in flight and about the
// number of vector-memory instructions, not about the matrix core.  Two kernels:
//
//  * fp8_gemm_transpose_kernel (M <= 32, K >= 1024): the weight rows are dealt out evenly over one block per
//    compute unit; a block's wavefronts take interleaved pairs of K-blocks, fetch them in runs of 256 bytes per
//    row and transpose them into MFMA operand layout through wavefront-private LDS slabs (see the kernel).
//  * fp8_gemm_smallm_kernel (the rest): work unit = (64 weight rows) x (one 128-byte K-block).  A wavefront
//    streams its units straight from global memory into registers: lane l owns weight row (l & 15) of each of
//    the four 16-row groups and the K bytes [16g, 16g+16) and [64+16g, 64+16g+16), g = l >> 4 -- the MFMA
//    operand layout, so no LDS staging is needed; the tiny activation fragment is fetched the same way (it stays
//    in L2).  The next unit's loads are issued before the current unit is multiplied.
//
// In both, the wavefronts of a block add their fp32 results in LDS.  When the chunks of rows do not give enough
// blocks to cover the GPU, several blocks split K.  Each writes an fp32 partial tile to the workspace; the block
// that arrives last (a counter per chunk) adds the partials in split order -- a fixed order, so results do not
// depend on timing -- and resets the counter, so the workspace needs zeroing only once, when it is allocated.
//
// Arithmetic follows the tile kernel: per K-block products accumulated by the fp8 MFMA, multiplied by
// As[m, kb] * Bs[n / 128, kb] in fp32 (block mode) or accumulated unscaled and scaled per row and column
// at the end (row/column mode).

#include "fp8_gemm_common.h"

#include <algorithm>

namespace fg {
namespace {

constexpr int kChunkRows = 64;  // weight rows per block
constexpr int kRowGroups = 4;   // 16-row MFMA groups per chunk

struct SmallArgs {
  GemmArgs g;
  int kpw, splits, n_chunks;
  // staged kernels: chunk c owns rows_lo + (c < rows_rem) weight rows, the chunks in ascending row order; the
  // activations of the block's K range are kept in LDS with rows x_lds_stride bytes apart (0: not kept)
  int rows_lo, rows_rem, x_lds_stride;
  int pw_pairs;  // pairs of K-blocks of the blocks that have most (per-wavefront form of the activations in LDS)
  int m_recip;  // 65535 / M + 1: (u * m_recip) >> 16 == u / M for the small u the kernel divides
  float* partials;      // [n_chunks][splits][16 * TMX][64]
  unsigned int* counters;
  int64_t partials_per_entry;  // floats; a batch (g.batch > 1, entry = blockIdx.y) keeps one such array and n_chunks counters per entry
};

// z-th problem of a batch: operands, partial sums and counters of that entry
__device__ __forceinline__ void select_batch_entry(SmallArgs& a, int64_t z) {
  if (a.g.batch > 1) {  // uniform
    a.g.X += z * a.g.x_batch_bytes;
    a.g.W += z * a.g.w_batch_bytes;
    a.g.C = reinterpret_cast<uint8_t*>(a.g.C) + z * a.g.c_batch_bytes;
    a.g.xs += z * a.g.xs_batch_stride;
    a.g.ws += z * a.g.ws_batch_stride;
    if (a.partials) a.partials += z * a.partials_per_entry;
    if (a.counters) a.counters += z * a.n_chunks;
    if (z == a.g.batch - 1) {  // parts of one problem's rows: the last part ends with the last row
      a.g.X -= a.g.last_x_back_bytes;
      a.g.C = reinterpret_cast<uint8_t*>(a.g.C) - a.g.last_c_back_bytes;
      a.g.xs -= a.g.last_xs_back;
    }
  }
}

__device__ __forceinline__ v8i join(u32x4 lo, u32x4 hi) {
  v8i f;
  f[0] = (int)lo.x; f[1] = (int)lo.y; f[2] = (int)lo.z; f[3] = (int)lo.w;
  f[4] = (int)hi.x; f[5] = (int)hi.y; f[6] = (int)hi.z; f[7] = (int)hi.w;
  return f;
}

template <int TMX>
struct Unit {  // operands of one K-block
  u32x4 wlo[kRowGroups], whi[kRowGroups];
  u32x4 xlo[TMX], xhi[TMX];
  float xs[TMX];
  float ws;
};

template <int TMX, int MODE>
__device__ __forceinline__ void load_unit(Unit<TMX>& u, const SmallArgs& a, const uint8_t* const (&wrow)[kRowGroups],
                                          const uint8_t* const (&xrow)[TMX], const float* const (&xsrow)[TMX],
                                          const float* wsrow, int kb) {
  const int64_t k = (int64_t)kb * 128;
#pragma unroll
  for (int r = 0; r < kRowGroups; ++r) {
    u.wlo[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[r] + k));
    u.whi[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[r] + k + 64));
  }
#pragma unroll
  for (int t = 0; t < TMX; ++t) {
    u.xlo[t] = *reinterpret_cast<const u32x4*>(xrow[t] + k);
    u.xhi[t] = *reinterpret_cast<const u32x4*>(xrow[t] + k + 64);
    if (MODE == kModeBlock) u.xs[t] = xsrow[t][(int64_t)kb * a.g.xs_cs];
  }
  if (MODE == kModeBlock) u.ws = wsrow[(int64_t)kb * a.g.ws_cs];
}

template <int TMX, int MODE>
__device__ __forceinline__ void compute_unit(const Unit<TMX>& u, v4f (&acc)[kRowGroups][TMX]) {
#pragma unroll
  for (int t = 0; t < TMX; ++t) {
    const v8i xf = join(u.xlo[t], u.xhi[t]);
    const float sc = (MODE == kModeBlock) ? u.xs[t] * u.ws : 1.f;
#pragma unroll
    for (int r = 0; r < kRowGroups; ++r) {
      const v8i wf = join(u.wlo[r], u.whi[r]);
      if (MODE == kModeBlock) {
        const v4f p = mfma_fp8_16x16x128(wf, xf, v4f{0.f, 0.f, 0.f, 0.f});
        acc[r][t][0] = __builtin_fmaf(p[0], sc, acc[r][t][0]);
        acc[r][t][1] = __builtin_fmaf(p[1], sc, acc[r][t][1]);
        acc[r][t][2] = __builtin_fmaf(p[2], sc, acc[r][t][2]);
        acc[r][t][3] = __builtin_fmaf(p[3], sc, acc[r][t][3]);
      } else {
        acc[r][t] = MODE == kModeRowColI8 ? mfma_i8_16x16x128(wf, xf, acc[r][t]) : mfma_fp8_16x16x128(wf, xf, acc[r][t]);
      }
    }
  }
}

// Sum of two partial results: fp32, or int32 bit patterns (int8 operands, whose sums stay exact).
__device__ __forceinline__ float add_partial(float a, float b, bool as_int) {
  return as_int ? __int_as_float(__float_as_int(a) + __float_as_int(b)) : a + b;
}

// Adds the wavefronts' accumulators in LDS and writes the chunk (or publishes a split-K partial tile and,
// in the block that arrives last, adds the partial tiles in split order).  Wavefront w's sums go to red[w * red_stride + m * 16*RG + n]; the chunk is
// rows n0 .. n0 + rows - 1.
template <int TMX, int RG, int WAVES, int MODE>
__device__ __forceinline__ void finish_chunk(const SmallArgs& a, float* red, int red_stride, int* last_flag,
                                             const v4f (&acc)[RG][TMX], int chunk, int split, int n0, int rows) {
  constexpr int NT = WAVES * 64;
  constexpr int MROWS = 16 * TMX;
  constexpr int kChunkRows = 16 * RG;
  constexpr int kRowGroups = RG;
  constexpr int kOut = MROWS * kChunkRows;
  const GemmArgs& g = a.g;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lg = lane >> 4;
  // bf16 results of the block-scaled product, the case these kernels meet in practice, are stored by a few
  // instructions of their own: the general epilogue is a long chain of branches, and at the end of a launch of a few
  // microseconds every instruction line it fetches is waited for by the whole GPU
  const bool plain = MODE == kModeBlock && g.c_dtype == FG_BF16;
  constexpr bool as_int = MODE == kModeRowColI8;
  // lane holds m = t*16 + l16, n = r*16 + 4*lg + [0,4)
#pragma unroll
  for (int r = 0; r < kRowGroups; ++r)
#pragma unroll
    for (int t = 0; t < TMX; ++t)
      *reinterpret_cast<v4f*>(red + wave * red_stride + ((t * 16 + l16) * kChunkRows + r * 16 + lg * 4)) = acc[r][t];
  __syncthreads();

  if (a.splits == 1) {
    for (int i = tid; i < kOut; i += NT) {
      const int m = i / kChunkRows, nn = i % kChunkRows;
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) v = add_partial(v, red[w * red_stride + i], as_int);
      if (m < g.M && nn < rows) {
        if (plain) reinterpret_cast<uint16_t*>(g.C)[(int64_t)m * g.ldc + n0 + nn] = float_to_bf16_bits(v);
        else store_output<MODE>(g, m, n0 + nn, v);
      }
    }
    return;
  }

  float* const mine = a.partials + ((int64_t)chunk * a.splits + split) * kOut;
  for (int i = tid; i < kOut; i += NT) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) v = add_partial(v, red[w * red_stride + i], as_int);
    // device-scope store: written through to memory, where blocks on other XCDs (own L2 each) read it
    __hip_atomic_store(mine + i, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // A device-scope fence here would write back and invalidate the whole L2 (measured ~50 us per
  // launch).  The partial tiles bypass the L2 on both sides instead, so it is enough that every
  // store of this block has been acknowledged before the counter moves: every thread waits for its
  // own stores (a workgroup-scope fence emits no such wait), then the barrier collects the block.
  wait_vmem_all();
  __syncthreads();
  if (tid == 0) {
    const unsigned int prev = __hip_atomic_fetch_add(&a.counters[chunk], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *last_flag = (prev == (unsigned int)(a.splits - 1)) ? 1 : 0;
  }
  __syncthreads();
  if (!*last_flag) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  const float* const all = a.partials + (int64_t)chunk * a.splits * kOut;
  for (int i = tid; i < kOut; i += NT) {
    const int m = i / kChunkRows, nn = i % kChunkRows;
    float v = 0.f;
    for (int s = 0; s < a.splits; ++s)
      v = add_partial(v, __hip_atomic_load(all + (int64_t)s * kOut + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), as_int);
    if (m < g.M && nn < rows) {
      if (plain) reinterpret_cast<uint16_t*>(g.C)[(int64_t)m * g.ldc + n0 + nn] = float_to_bf16_bits(v);
      else store_output<MODE>(g, m, n0 + nn, v);
    }
  }
  if (tid == 0) __hip_atomic_store(&a.counters[chunk], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
}

template <int TMX, int WAVES, int MODE>
__global__ __launch_bounds__(WAVES * 64) void fp8_gemm_smallm_kernel(SmallArgs a) {
  constexpr int MROWS = 16 * TMX;
  __shared__ float red[WAVES][MROWS][kChunkRows];  // 4 KB * TMX per wavefront
  __shared__ int last_flag;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  select_batch_entry(a, blockIdx.y);
  const int chunk = blockIdx.x % a.n_chunks;
  const int split = blockIdx.x / a.n_chunks;
  const int n0 = chunk * kChunkRows;
  const int l16 = lane & 15, lg = lane >> 4;
  const GemmArgs& g = a.g;

  // row pointers of this lane (rows past the edge alias the last valid row; never stored)
  const uint8_t* wrow[kRowGroups];
#pragma unroll
  for (int r = 0; r < kRowGroups; ++r) {
    int n = n0 + r * 16 + l16;
    n = n < g.N ? n : g.N - 1;
    wrow[r] = g.W + (int64_t)n * g.ldw + lg * 16;
  }
  const uint8_t* xrow[TMX];
  const float* xsrow[TMX];
#pragma unroll
  for (int t = 0; t < TMX; ++t) {
    int m = t * 16 + l16;
    m = m < g.M ? m : g.M - 1;
    xrow[t] = g.X + (int64_t)m * g.ldx + lg * 16;
    xsrow[t] = (MODE == kModeBlock) ? g.xs + (int64_t)m * g.xs_rs : nullptr;
  }
  const float* wsrow = (MODE == kModeBlock) ? g.ws + (int64_t)(n0 >> 7) * g.ws_rs : nullptr;

  v4f acc[kRowGroups][TMX];
#pragma unroll
  for (int r = 0; r < kRowGroups; ++r)
#pragma unroll
    for (int t = 0; t < TMX; ++t) acc[r][t] = v4f{0.f, 0.f, 0.f, 0.f};

  // K-blocks of this wavefront: kb = first + i * WAVES, i < kpw, inside this split's range
  const int per_split = a.kpw * WAVES;
  const int kb_end = min(g.KB, (split + 1) * per_split);
  int kb = split * per_split + wave;
  if (kb < kb_end) {
    Unit<TMX> cur;
    load_unit<TMX, MODE>(cur, a, wrow, xrow, xsrow, wsrow, kb);
    for (kb += WAVES; kb < kb_end; kb += WAVES) {
      Unit<TMX> nxt;
      load_unit<TMX, MODE>(nxt, a, wrow, xrow, xsrow, wsrow, kb);
      compute_unit<TMX, MODE>(cur, acc);
      cur = nxt;
    }
    compute_unit<TMX, MODE>(cur, acc);
  }

  finish_chunk<TMX, kRowGroups, WAVES, MODE>(a, &red[0][0][0], MROWS * kChunkRows, &last_flag, acc, chunk, split, n0, min(kChunkRows, g.N - n0));
}

// ---------------------------------------------------------------------------------------------
// Transposing variant (M <= 32, K >= 1024, and wide weights from K = 256 on).  The weight bytes are fetched in
// runs of 256 contiguous bytes per row (two K-blocks; 4 rows per wavefront load instruction) instead
// of the 64-byte pieces the MFMA operand layout dictates: measured on MI355X a pure load of a
// [7168, 16384] matrix reaches 5.8 TB/s with 256-byte runs against 5.0 TB/s with 64-byte pieces, and of a
// [2112, 7168] matrix with this kernel's ownership 3.6 against 2.5 TB/s.  The loads land in registers; when a
// pair of K-blocks has arrived the wavefront writes it to its private LDS slab (4 KB per 16 rows) and reads it
// back in operand layout.  No barrier is involved before the final reduction: a wavefront's LDS operations
// execute in order.  Within a row the sixteen 16-byte chunks are permuted (physical chunk p holds
// logical chunk p ^ (row & 15)) so that both the writes (4 rows x 256 B) and the operand reads (16 rows
// 256 bytes apart) spread over all LDS banks.
// ---------------------------------------------------------------------------------------------
template <int TMX, int Q>
struct PairRegs {
  u32x4 w[Q];                  // load j: rows 4j..4j+3, lane -> row 4j + (l >> 4), bytes 16*(l & 15) of the pair
  u32x4 xlo[2][TMX], xhi[2][TMX];  // the last three only when the activations do not come from LDS
  float xs[2][TMX];
  float wsv;                   // lane & 3 -> weight scale of K-block (lane & 1) of the pair in scale block (lane >> 1) & 1 of the chunk
};

// Global -> LDS copies the compiler does not see: 16 (4) bytes per lane to lds_addr + 16 (4) * lane.  `base` and
// `lds_addr` are wave-uniform; the copies count in vmcnt like loads and complete in order with them.
__device__ __forceinline__ void dma_to_lds_16(uint32_t byte_off, const void* base, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(byte_off), "s"(base), "s"(lds_addr) : "memory", "m0");
}
__device__ __forceinline__ void dma_to_lds_4(uint32_t byte_off, const void* base, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" : : "v"(byte_off), "s"(base), "s"(lds_addr) : "memory", "m0");
}

// Q = 4-row groups of weights per chunk (a chunk has up to 4Q rows, the block's wavefronts take interleaved pairs
// of K-blocks), DEPTH = K-block pairs in flight per wavefront.
//
// A launch of a few microseconds is bound by what a compute unit does around its bytes: every vector-memory
// instruction occupies the address unit (about 14 cycles each, whatever it carries), and a wavefront that issues a
// load while the memory pipeline is full blocks at the issue.  So, when XLDS is set (M <= 16), nothing but weights is
// loaded per pair of K-blocks: at its start every wavefront copies the activations its own pairs need, their scales
// and the weight scales into LDS with a handful of global -> LDS copies (no barrier: a pair is multiplied by the
// wavefront that copied for it, and the wait for its first weights is also the wait for its copies, which were
// issued earlier and complete in order); the ring holds one pair, whose refill goes out as soon as it is in the slab,
// and the chunk has no more 4-row groups than its rows need.  RING: the activations of a wavefront's pairs do not
// fit LDS all at once (M = 16 with K of 7168 and more), so it keeps two slots and copies for pair i + 1 after pair i
// is in the slab and before the refill goes out: the wait for the refilled weights is again the wait for the copies.
// OWN (wide weights): every wavefront has a chunk of
// its own and walks all of K, so the block shares the activations (one barrier) and nothing is added across
// wavefronts.  Without XLDS (activations too large for LDS, or too few pairs per wavefront to pay for the copies)
// the activation fragments travel in the register ring next to the weights.
template <int TMX, int Q, int DEPTH, int WAVES, int MODE, bool XLDS, bool OWN = false, bool RING = false>
__global__ __launch_bounds__(WAVES * 64) void fp8_gemm_transpose_kernel(SmallArgs a) {
  static_assert(!XLDS || TMX == 1 || OWN, "activations in LDS: M <= 16, or more rows where the block shares them");
  static_assert(!OWN || XLDS, "wavefronts with chunks of their own share the activations through LDS");
  static_assert(!RING || (XLDS && !OWN && DEPTH == 1), "the two-slot form belongs to the per-wavefront copies with one pair in the ring");
  constexpr int RG = (Q + 3) / 4;
  constexpr int kRows = 16 * RG;
  constexpr int kSlab = kRows * 256;  // one K-block pair of the chunk
  constexpr int NT = WAVES * 64;
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];  // WAVES slabs (later the reduction buffer), activations, scales
  __shared__ int last_flag;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, lg = lane >> 4;
  const GemmArgs& g = a.g;
  const int64_t z = blockIdx.z;  // batch entry
  const int split = blockIdx.y;
  // OWN: every wavefront has a chunk of its own and walks all of K (nothing is added across wavefronts); the last
  // block may have wavefronts without a chunk, which still help to copy the activations
  const int chunk = OWN ? min((int)blockIdx.x * WAVES + wave, a.n_chunks - 1) : (int)blockIdx.x;
  const bool idle = OWN && (int)blockIdx.x * WAVES + wave >= a.n_chunks;
  const int n0 = chunk * a.rows_lo + min(chunk, a.rows_rem);
  const int rows_valid = a.rows_lo + (chunk < a.rows_rem ? 1 : 0);  // 1 .. 4Q
  uint8_t* const slab = lds + wave * kSlab;

  const int pairs_total = (g.KB + 1) >> 1;
  const int pair_lo = OWN ? 0 : split * a.kpw * WAVES;
  const int pair_end = OWN ? pairs_total : min(pairs_total, pair_lo + a.kpw * WAVES);
  const int kb_lo = pair_lo * 2;
  const int kbc = min(g.KB, pair_end * 2) - kb_lo;  // K-blocks of this block

  const bool last_entry = g.batch > 1 && z == g.batch - 1;  // uniform
  const uint8_t* const x_base = g.X + z * g.x_batch_bytes - (last_entry ? g.last_x_back_bytes : 0);
  const float* const xs_base = (MODE == kModeBlock) ? g.xs + z * g.xs_batch_stride - (last_entry ? g.last_xs_back : 0) : nullptr;
  const uint32_t xs_cs = (uint32_t)g.xs_cs;

  // weight scales: a chunk may begin anywhere, so its rows can lie in two 128-row scale blocks; second[r][i] says
  // that this lane's column r*16 + 4*lg + i belongs to the second (lane masks, set up once).
  const float* const ws_base =
      (MODE == kModeBlock) ? g.ws + z * g.ws_batch_stride + (int64_t)(n0 >> 7) * g.ws_rs : nullptr;
  const int64_t ws_second = (((n0 + rows_valid - 1) >> 7) != (n0 >> 7)) ? g.ws_rs : 0;
  bool second[RG][4];
#pragma unroll
  for (int r = 0; r < RG; ++r)
#pragma unroll
    for (int i = 0; i < 4; ++i) second[r][i] = ((n0 + r * 16 + lg * 4 + i) >> 7) != (n0 >> 7);


  // ---- activations and their scales -> LDS (issued before the first weight load: they arrive first)
  constexpr bool PW = XLDS && !OWN;  // every wavefront copies what its own pairs of K-blocks need: no barrier
  // RING: a wavefront keeps two slots only and copies pair i + 1 while it multiplies pair i (activations of the whole
  // K range too large for LDS)
  const uint32_t lds_x = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds + WAVES * kSlab;
  // shared form (OWN): rows x_lds_stride apart, 16-byte pieces permuted; [M][kbc] activation scales; [2][kbc] weight
  // scales per wavefront
  const uint32_t x_stride = (uint32_t)a.x_lds_stride;
  const uint32_t lds_xs = lds_x + (uint32_t)g.M * x_stride;
  const uint32_t lds_ws = lds_xs + (uint32_t)(g.M * kbc) * 4u + (uint32_t)(wave * 2 * kbc) * 4u;
  // per-wavefront form (PW): slot i of a wavefront is its i-th pair; [slot][row][256 B] activations with the 16
  // pieces of a row's pair permuted by the row, [slot][K-block][row] activation scales, [slot][scale block][K-block]
  // weight scales
  // (the block's pairs are dealt round-robin, so wavefront w's slots begin after those of the wavefronts before it)
  const int blk_pairs = pair_end - pair_lo;
  const uint32_t slot0 = RING ? (uint32_t)(wave * 2) : (uint32_t)(wave * (blk_pairs / WAVES) + min(wave, blk_pairs % WAVES));
  const uint32_t pw_x = lds_x + slot0 * (uint32_t)g.M * 256u;
  const uint32_t pw_xs = lds_x + (uint32_t)(a.pw_pairs * g.M) * 256u + slot0 * (uint32_t)(2 * g.M) * 4u;
  const uint32_t pw_ws = lds_x + (uint32_t)(a.pw_pairs * g.M) * (256u + 8u) + slot0 * 16u;
  // RING: the i-th pair of this wavefront -> slot i & 1 (same layout as below, one pair at a time)
  auto copy_pair = [&](int i) __attribute__((always_inline)) {
    const int p = pair_lo + wave + i * WAVES;
    const uint32_t s = (uint32_t)(i & 1);
    const bool two = p * 2 + 1 < g.KB;
    for (int j = 0; j * 4 < g.M; ++j) {
      const int m = j * 4 + lg;
      if (m < g.M) {
        int piece = l16 ^ (m & 15);
        if (!two && piece >= 8) piece -= 8;
        dma_to_lds_16((uint32_t)m * (uint32_t)g.ldx + (uint32_t)p * 256u + (uint32_t)piece * 16u, x_base,
                      pw_x + s * (uint32_t)g.M * 256u + (uint32_t)j * 1024u);
      }
    }
    if (MODE == kModeBlock) {
      if (lane < 2 * g.M) {  // lane = b * M + row
        const int b = lane >= g.M ? 1 : 0, m = lane - b * g.M;
        const int kb = p * 2 + ((b && two) ? 1 : 0);
        dma_to_lds_4(((uint32_t)m * (uint32_t)g.xs_rs + (uint32_t)kb * xs_cs) * 4u, xs_base, pw_xs + s * (uint32_t)(2 * g.M) * 4u);
      }
      if (lane < 4) {  // lane = scale block * 2 + b
        const int kb = p * 2 + (((lane & 1) && two) ? 1 : 0);
        dma_to_lds_4((uint32_t)((int64_t)kb * g.ws_cs + ((lane & 2) ? ws_second : 0)) * 4u, ws_base, pw_ws + s * 16u);
      }
    }
  };
  if (RING) {
    if (pair_lo + wave < pair_end) copy_pair(0);
  } else if (PW) {
    const int first = pair_lo + wave;
    const int my_pairs = first < pair_end ? (pair_end - first + WAVES - 1) / WAVES : 0;
    const int recip = a.m_recip;
    // one copy = 4 (slot, row) units of 256 bytes; physical piece l16 of a unit holds logical piece l16 ^ (row & 15),
    // so that the 16 rows a wavefront reads together fall into 16 different 16-byte bank groups.  Where the pair's
    // second K-block does not exist its pieces repeat the first's.
    const int units = my_pairs * g.M;
    for (int j = 0; j * 4 < units; ++j) {
      const int u = j * 4 + lg;
      if (u < units) {
        const int i = (u * recip) >> 16, m = u - i * g.M;
        const int p = first + i * WAVES;
        int piece = l16 ^ (m & 15);
        if (p * 2 + 1 >= g.KB && piece >= 8) piece -= 8;
        dma_to_lds_16((uint32_t)m * (uint32_t)g.ldx + (uint32_t)p * 256u + (uint32_t)piece * 16u, x_base, pw_x + (uint32_t)j * 1024u);
      }
    }
    if (MODE == kModeBlock) {
      const int count = my_pairs * 2 * g.M;  // e = (slot * 2 + b) * M + row
      for (int j = 0; j * 64 < count; ++j) {
        const int e = j * 64 + lane;
        if (e < count) {
          const int q = (e * recip) >> 16, m = e - q * g.M;
          const int p = first + (q >> 1) * WAVES;
          const int kb = p * 2 + (((q & 1) && p * 2 + 1 < g.KB) ? 1 : 0);
          dma_to_lds_4(((uint32_t)m * (uint32_t)g.xs_rs + (uint32_t)kb * xs_cs) * 4u, xs_base, pw_xs + (uint32_t)j * 256u);
        }
      }
      const int wcount = my_pairs * 4;  // e = slot * 4 + scale block * 2 + b
      for (int j = 0; j * 64 < wcount; ++j) {
        const int e = j * 64 + lane;
        if (e < wcount) {
          const int p = first + (e >> 2) * WAVES;
          const int kb = p * 2 + (((e & 1) && p * 2 + 1 < g.KB) ? 1 : 0);
          dma_to_lds_4((uint32_t)((int64_t)kb * g.ws_cs + ((e & 2) ? ws_second : 0)) * 4u, ws_base, pw_ws + (uint32_t)j * 256u);
        }
      }
    }
  }
  if (XLDS && OWN) {
    // one copy = 64 pieces of 16 bytes of one row; piece p of a row lies at position p ^ perm(row) within its
    // K-block (8 pieces), perm(row) = (row >> 1) & 7, and the row stride is an odd multiple of 128 bytes: the 16
    // rows a wavefront reads together then fall into 16 different 16-byte bank groups
    const int row_pieces = kbc * 8;
    const int row_units = (row_pieces + 63) >> 6;
    const int units = g.M * row_units;
    int m = 0, ru = wave;
    while (ru >= row_units) { ru -= row_units; ++m; }
    for (int u = wave; u < units; u += WAVES) {
      const int p = ru * 64 + lane;
      if (p < row_pieces) {
        const uint32_t src = (uint32_t)m * (uint32_t)g.ldx + (uint32_t)kb_lo * 128u +
                             (uint32_t)(((p & ~7) | ((p & 7) ^ ((m >> 1) & 7))) << 4);
        dma_to_lds_16(src, x_base, lds_x + (uint32_t)m * x_stride + (uint32_t)ru * 1024u);
      }
      ru += WAVES;
      while (ru >= row_units) { ru -= row_units; ++m; }
    }
    if (MODE == kModeBlock) {
      const int count = g.M * kbc;
      for (int e0 = wave * 64; e0 < count; e0 += NT) {
        const int e = e0 + lane;
        if (e < count) {
          const int mm = e / kbc, kk = e - mm * kbc;
          dma_to_lds_4(((uint32_t)mm * (uint32_t)g.xs_rs + (uint32_t)(kb_lo + kk) * xs_cs) * 4u, xs_base, lds_xs + (uint32_t)e0 * 4u);
        }
      }
    }
    if (MODE == kModeBlock) {
      const int row_units = (kbc + 63) >> 6;
      for (int c = 0; c < 2 * row_units; ++c) {
        const int row = c & 1, k0 = (c >> 1) * 64;
        if (k0 + lane < kbc)
          dma_to_lds_4((uint32_t)((int64_t)(kb_lo + k0 + lane) * g.ws_cs + (row ? ws_second : 0)) * 4u, ws_base,
                       lds_ws + (uint32_t)(row * kbc + k0) * 4u);
      }
    }
  }

  // ---- weights: rows 4j + lg of the chunk, 16 bytes at l16 * 16 of the pair (rows past the chunk's last alias it;
  // never stored); a uniform 64-bit base plus 32-bit lane offsets
  const uint8_t* const w_base = g.W + z * g.w_batch_bytes + (int64_t)n0 * g.ldw;
  uint32_t w_off[Q];
#pragma unroll
  for (int j = 0; j < Q; ++j) {
    int r = 4 * j + lg;
    r = r < rows_valid ? r : rows_valid - 1;
    w_off[j] = (uint32_t)r * (uint32_t)g.ldw + (uint32_t)l16 * 16u;
  }
  // an odd K-block count leaves a single block at the end: lanes 8..15 of a row, which own the second K-block of
  // a pair, re-read the first
  const uint32_t tail_adj = l16 >= 8 ? 0xFFFFFF80u : 0u;

  // activation fragments of this lane: row t*16 + l16 (rows past M alias the last; never stored)
  uint32_t x_off[TMX], xs_off[TMX], lds_xrow[TMX], lds_xsrow[TMX];
#pragma unroll
  for (int t = 0; t < TMX; ++t) {
    int m = t * 16 + l16;
    m = m < g.M ? m : g.M - 1;
    x_off[t] = (uint32_t)m * (uint32_t)g.ldx + (uint32_t)lg * 16u;
    xs_off[t] = (uint32_t)m * (uint32_t)g.xs_rs;
    lds_xrow[t] = lds_x + (uint32_t)m * x_stride;
    lds_xsrow[t] = lds_xs + (uint32_t)(m * kbc) * 4u;
  }
  const uint32_t mrow = (uint32_t)(l16 < g.M ? l16 : g.M - 1);  // per-wavefront copies: TMX == 1
  const uint32_t perm = mrow & 15u;
  // shared form: where this lane's two pieces of a K-block lie in row t * 16 + l16 (see the copies above)
  uint32_t x_lo_piece[TMX], x_hi_piece[TMX];
#pragma unroll
  for (int t = 0; t < TMX; ++t) {
    int m = t * 16 + l16;
    m = m < g.M ? m : g.M - 1;
    const uint32_t pm = ((uint32_t)m >> 1) & 7u;
    x_lo_piece[t] = ((uint32_t)lg ^ pm) << 4;
    x_hi_piece[t] = ((uint32_t)(lg + 4) ^ pm) << 4;
  }
  int slot = 0;  // PW: index of the pair among this wavefront's

  v4f acc[RG][TMX];
#pragma unroll
  for (int r = 0; r < RG; ++r)
#pragma unroll
    for (int t = 0; t < TMX; ++t) acc[r][t] = v4f{0.f, 0.f, 0.f, 0.f};

  auto load_w = [&](PairRegs<TMX, Q>& u, int pair) __attribute__((always_inline)) {
    const bool two = pair * 2 + 1 < g.KB;
    const uint8_t* const base = w_base + (uint32_t)pair * 256u;
    const uint32_t adj = two ? 0u : tail_adj;
#pragma unroll
    for (int j = 0; j < Q; ++j)
      u.w[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + (size_t)(w_off[j] + adj)));
  };
  auto load_x = [&](PairRegs<TMX, Q>& u, int pair) __attribute__((always_inline)) {
    if (XLDS) return;
    const int kb = pair * 2;
    const bool two = kb + 1 < g.KB;
    if (MODE == kModeBlock) u.wsv = ws_base[(int64_t)(kb + ((two && (lane & 1)) ? 1 : 0)) * g.ws_cs + ((lane & 2) ? ws_second : 0)];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const uint32_t kbb = (uint32_t)(kb + ((b == 1 && two) ? 1 : 0));
      const uint8_t* const base = x_base + kbb * 128u;
#pragma unroll
      for (int t = 0; t < TMX; ++t) {
        u.xlo[b][t] = *reinterpret_cast<const u32x4*>(base + (size_t)x_off[t]);
        u.xhi[b][t] = *reinterpret_cast<const u32x4*>(base + (size_t)(x_off[t] + 64u));
        if (MODE == kModeBlock) u.xs[b][t] = xs_base[(size_t)(xs_off[t] + kbb * xs_cs)];
      }
    }
  };

  // registers -> slab: row R = 4j + lg, logical chunk l16 goes to physical chunk l16 ^ (R & 15)
  auto stage = [&](const PairRegs<TMX, Q>& u) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < Q; ++j) {
      const int R = 4 * j + lg;
      *reinterpret_cast<u32x4*>(slab + R * 256 + ((l16 ^ (R & 15)) << 4)) = u.w[j];
    }
  };
  // slab -> operand fragments: lane owns row rg*16 + l16 and logical chunks b*8 + lg, b*8 + lg + 4
  auto multiply = [&](const PairRegs<TMX, Q>& u, int pair) __attribute__((always_inline)) {
    const int kb = pair * 2;
    const bool two = kb + 1 < g.KB;
    const int rs = RING ? (slot & 1) : slot;  // where this pair's activations and scales lie
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      if (b == 1 && !two) break;
      float ws1 = 1.f, ws2 = 1.f;
      if (MODE == kModeBlock) {
        if (PW) {
          ws1 = *reinterpret_cast<const __attribute__((address_space(3))) float*>(pw_ws + (uint32_t)(rs * 4 + b) * 4u);
          ws2 = *reinterpret_cast<const __attribute__((address_space(3))) float*>(pw_ws + (uint32_t)(rs * 4 + 2 + b) * 4u);
        } else if (XLDS) {
          ws1 = *reinterpret_cast<const __attribute__((address_space(3))) float*>(lds_ws + (uint32_t)(kb + b - kb_lo) * 4u);
          ws2 = *reinterpret_cast<const __attribute__((address_space(3))) float*>(lds_ws + (uint32_t)(kbc + kb + b - kb_lo) * 4u);
        } else {
          ws1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, u.wsv), b));
          ws2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, u.wsv), 2 + b));
        }
      }
      v8i xf[TMX];
      float xsc[TMX];
#pragma unroll
      for (int t = 0; t < TMX; ++t) {
        if (PW) {
          // the pair's 16 pieces are permuted as a whole: logical piece b*8 + lg (+4) sits at that number ^ perm
          const uint32_t at = pw_x + ((uint32_t)(rs * g.M) + mrow) * 256u;
          const u32x4 lo = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(at + (((uint32_t)(b * 8 + lg) ^ perm) << 4));
          const u32x4 hi = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(at + (((uint32_t)(b * 8 + lg + 4) ^ perm) << 4));
          xf[t] = join(lo, hi);
          xsc[t] = (MODE == kModeBlock)
                       ? *reinterpret_cast<const __attribute__((address_space(3))) float*>(pw_xs + ((uint32_t)((rs * 2 + b) * g.M) + mrow) * 4u)
                       : 1.f;
        } else if (XLDS) {
          const uint32_t at = lds_xrow[t] + (uint32_t)(kb + b - kb_lo) * 128u;
          const u32x4 lo = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(at + x_lo_piece[t]);
          const u32x4 hi = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(at + x_hi_piece[t]);
          xf[t] = join(lo, hi);
          xsc[t] = (MODE == kModeBlock)
                       ? *reinterpret_cast<const __attribute__((address_space(3))) float*>(lds_xsrow[t] + (uint32_t)(kb + b - kb_lo) * 4u)
                       : 1.f;
        } else {
          xf[t] = join(u.xlo[b][t], u.xhi[b][t]);
          xsc[t] = (MODE == kModeBlock) ? u.xs[b][t] : 1.f;
        }
      }
#pragma unroll
      for (int r = 0; r < RG; ++r) {
        const uint8_t* row = slab + (r * 16 + l16) * 256;
        const u32x4 lo = *reinterpret_cast<const u32x4*>(row + (((b * 8 + lg) ^ l16) << 4));
        const u32x4 hi = *reinterpret_cast<const u32x4*>(row + (((b * 8 + lg + 4) ^ l16) << 4));
        const v8i wf = join(lo, hi);
#pragma unroll
        for (int t = 0; t < TMX; ++t) {
          if (MODE == kModeBlock) {
            const float sc1 = xsc[t] * ws1, sc2 = xsc[t] * ws2;
            const v4f p = mfma_fp8_16x16x128(wf, xf[t], v4f{0.f, 0.f, 0.f, 0.f});
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[r][t][i] = __builtin_fmaf(p[i], second[r][i] ? sc2 : sc1, acc[r][t][i]);
          } else {
            acc[r][t] = MODE == kModeRowColI8 ? mfma_i8_16x16x128(wf, xf[t], acc[r][t]) : mfma_fp8_16x16x128(wf, xf[t], acc[r][t]);
          }
        }
      }
    }
  };

  // DEPTH register sets form a ring; the loop body is written out once per set so that the ring index is static
  // and nothing is copied between sets.
  constexpr int STEP = OWN ? 1 : WAVES;
  int pair = OWN ? (idle ? pair_end : pair_lo) : pair_lo + wave;
  PairRegs<TMX, Q> ring[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (pair + d * STEP < pair_end) {
      load_w(ring[d], pair + d * STEP);
      load_x(ring[d], pair + d * STEP);
    }
  bool done = pair >= pair_end;
  bool staged_ahead = false;
  if (XLDS) {
    // The wait for the first pair of weights is also the wait for this wavefront's copies, which were issued
    // earlier and complete in order; a wavefront without work waits for its copies alone.
    if (!done) { stage(ring[0]); staged_ahead = true; }
    else wait_vmem_all();
    if (OWN) __syncthreads();
    else asm volatile("" ::: "memory");  // the reads of what the copies brought stay behind that wait
  }
  while (!done) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (!done) {
        const int refill = pair + DEPTH * STEP;
        if (d == 0 && staged_ahead) staged_ahead = false;
        else stage(ring[d]);
        // With the activations in LDS the ring holds weights only and its registers are free once they are in
        // the slab: the refill goes out before the multiplication, so the slab double-buffers the ring.  With
        // activation fragments in the ring the refill has to follow the multiplication.
        if (RING) {
          // the slot of pair i + 1 was last read by the multiplication of pair i - 1; its copies go out ahead of the
          // refill, so the wait for the refilled weights is the wait for them as well
          asm volatile("" ::: "memory");
          if (refill < pair_end) copy_pair(slot + 1);
        }
        if (XLDS && refill < pair_end) load_w(ring[d], refill);
        multiply(ring[d], pair);
        if (!XLDS && refill < pair_end) {
          load_w(ring[d], refill);
          load_x(ring[d], refill);
        }
        pair += STEP;
        ++slot;
        done = pair >= pair_end;
      }
    }
  }

  select_batch_entry(a, z);  // the epilogue's view of the operands
  if (OWN) {
    if (idle) return;
    // lane holds m = l16, n = n0 + r*16 + 4*lg + [0,4); bf16 results of the block-scaled product take a short path
    // of their own (see finish_chunk)
    const bool plain = MODE == kModeBlock && g.c_dtype == FG_BF16;
#pragma unroll
    for (int t = 0; t < TMX; ++t) {
      const int m = t * 16 + l16;
      uint16_t* const c_row = reinterpret_cast<uint16_t*>(g.C) + (int64_t)m * g.ldc + n0;
#pragma unroll
      for (int r = 0; r < RG; ++r)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int nn = r * 16 + lg * 4 + i;
          if (m < g.M && nn < rows_valid) {
            if (plain) c_row[nn] = float_to_bf16_bits(acc[r][t][i]);
            else store_output<MODE>(g, m, n0 + nn, acc[r][t][i]);
          }
        }
    }
    return;
  }
  // a wavefront's sums (16*TMX x 16*RG floats) go into its own slab, which only it has used: no barrier before them
  static_assert(16 * TMX * 4 <= 256, "a wavefront's sums fit its slab");
  finish_chunk<TMX, RG, WAVES, MODE>(a, reinterpret_cast<float*>(lds), kSlab / 4, &last_flag, acc, chunk, split, n0, rows_valid);
}

template <int TMX, int WAVES>
int launch_t(const SmallArgs& sa, int mode, hipStream_t stream) {
  const dim3 grid((uint32_t)(sa.n_chunks * sa.splits), (uint32_t)(sa.g.batch > 1 ? sa.g.batch : 1)), block(WAVES * 64);
  if (mode == kModeBlock) FG_LAUNCH((fp8_gemm_smallm_kernel<TMX, WAVES, kModeBlock>), grid, block, 0, stream, sa);
  else if (mode == kModeRowColI8) FG_LAUNCH((fp8_gemm_smallm_kernel<TMX, WAVES, kModeRowColI8>), grid, block, 0, stream, sa);
  else FG_LAUNCH((fp8_gemm_smallm_kernel<TMX, WAVES, kModeRowCol>), grid, block, 0, stream, sa);
  FG_CHECK_LAUNCH("fp8_gemm_smallm_kernel");
  return FG_OK;
}

constexpr int kDecodeLdsLimit = 160 * 1024 - 1024;  // dynamic LDS a block may ask for (a little is static)

// bytes between activation rows in LDS: the K-blocks of the block's range, an odd number of 128-byte units
inline int x_lds_stride_for(int64_t kbc) { return (int)((kbc | 1) * 128); }
// dynamic LDS of the staged kernel with the activations kept in LDS (weight scales counted once per wavefront,
// which only the kernel with a chunk per wavefront needs)
inline int64_t decode_lds_bytes(int q, int waves, int64_t M, int64_t kbc) {
  return (int64_t)waves * 16 * ((q + 3) / 4) * 256 + M * x_lds_stride_for(kbc) + (M + 2 * waves) * kbc * 4;
}
// the same with every wavefront keeping what its own pairs of K-blocks need; `pairs` = pairs of K-blocks per block
inline int64_t decode_lds_bytes_per_wave(int q, int waves, int64_t M, int64_t pairs) {
  return (int64_t)waves * 16 * ((q + 3) / 4) * 256 + pairs * (M * 256 + 2 * M * 4 + 16);
}

template <int TMX, int Q, int DEPTH, int WAVES, bool XLDS, bool OWN = false, bool RING = false>
int launch_transpose(const SmallArgs& sa, int mode, hipStream_t stream) {
  // WAVES slabs of 4 KB per 16 rows; the reduction buffer (WAVES * 16*TMX * rows floats) reuses the same memory
  constexpr int kSlabs = WAVES * 16 * ((Q + 3) / 4) * 256;
  const int64_t kbc = OWN ? sa.g.KB : std::min<int64_t>(sa.g.KB, (int64_t)sa.kpw * WAVES * 2);
  const int lds_bytes = !XLDS ? kSlabs : OWN ? (int)decode_lds_bytes(Q, WAVES, sa.g.M, kbc) : (int)decode_lds_bytes_per_wave(Q, WAVES, sa.g.M, sa.pw_pairs);
  if (lds_bytes > kDecodeLdsLimit) FG_FAIL(FG_ERR_LAUNCH, "fp8 gemm (small M): %d bytes of LDS planned", lds_bytes);
  const dim3 grid((uint32_t)(OWN ? ceil_div(sa.n_chunks, WAVES) : sa.n_chunks), (uint32_t)sa.splits, (uint32_t)(sa.g.batch > 1 ? sa.g.batch : 1));
  const dim3 block(WAVES * 64);
  auto kb = fp8_gemm_transpose_kernel<TMX, Q, DEPTH, WAVES, kModeBlock, XLDS, OWN, RING>;
  auto kr = fp8_gemm_transpose_kernel<TMX, Q, DEPTH, WAVES, kModeRowCol, XLDS, OWN, RING>;
  auto ki = fp8_gemm_transpose_kernel<TMX, Q, DEPTH, WAVES, kModeRowColI8, XLDS, OWN, RING>;
  static PerDeviceFlags lds_limit_raised = {};  // per instantiation
  {
    const hipError_t e = raise_dynamic_lds_limit(lds_limit_raised, XLDS ? kDecodeLdsLimit : kSlabs, reinterpret_cast<const void*>(kb), reinterpret_cast<const void*>(kr),
                                                  reinterpret_cast<const void*>(ki));
    if (e != hipSuccess) FG_FAIL(FG_ERR_LAUNCH, "hipFuncSetAttribute(LDS limit): %s", hipGetErrorString(e));
  }
  if (mode == kModeBlock) FG_LAUNCH(kb, grid, block, lds_bytes, stream, sa);
  else if (mode == kModeRowColI8) FG_LAUNCH(ki, grid, block, lds_bytes, stream, sa);
  else FG_LAUNCH(kr, grid, block, lds_bytes, stream, sa);
  FG_CHECK_LAUNCH("fp8_gemm_transpose_kernel");
  return FG_OK;
}

}  // namespace

SmallMPlan plan_small_m(int64_t M, int64_t N, int64_t K, int64_t entries) {
  if (entries < 1) entries = 1;  // equal problems launched together: their blocks fill the GPU together
  SmallMPlan p = {};
  p.use = false;
  if (M < 1 || M > 64 || N < 1 || K < 128 || K % 128 != 0) return p;
  p.tmx = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int64_t KB = K / 128;
  int64_t kpw, splits;
  p.rg = kRowGroups;
  p.q = 4 * kRowGroups;
  p.xlds = false;
  p.staged = p.tmx <= 2 && KB >= 8;
  int64_t chunks = 0;
  // One block per compute unit with the rows dealt out evenly (chunks differ by at most one row): a launch takes as
  // long as the compute unit with most bytes to fetch.  Narrow weights get chunks of at least `rows_min` rows and K
  // split over blocks below; weights with more than 64 rows per compute unit get whole rounds of blocks.
  const int64_t B = std::max<int64_t>(1, cu_count() / entries);
  auto deal_rows = [&](int64_t rows_min, int64_t blocks = 0) {
    if (blocks < 1) blocks = B;
    chunks = N <= 64 * blocks ? std::min<int64_t>(blocks, ceil_div(N, rows_min)) : ceil_div(N, 64 * blocks) * blocks;
    const int64_t rows_max = ceil_div(N, chunks);
    p.q = (int)ceil_div(rows_max, 4);
    p.rg = p.q <= 4 ? 1 : (p.q <= 8 ? 2 : 4);
    p.waves = (p.tmx == 2 && p.rg == 4) ? 4 : 8;
  };
  if (p.staged) {
    deal_rows(p.tmx == 1 ? 4 : 16);
  } else {
    p.waves = p.tmx == 4 ? 4 : 8;  // LDS reduction buffer is 4 KB * tmx per wavefront
  }
  p.n_chunks = p.staged ? (int)chunks : (int)ceil_div(N, 16 * p.rg);
  if (p.n_chunks > FG_WORKSPACE_COUNTER_BYTES / 4) return p;
  // partial tiles cost 2 * splits * 16*tmx * rows * 4 bytes per chunk against rows * K weight bytes: keep
  // them under a quarter of the weight traffic
  const int64_t max_splits = K / (32 * 16 * p.tmx) > 1 ? K / (32 * 16 * p.tmx) : 1;
  if (p.staged) {
    const int64_t pairs = (KB + 1) / 2;
    auto split_k = [&]() {
      p.n_chunks = (int)chunks;
      splits = 1;
      while (p.n_chunks * entries * splits < 100 && splits * 2 <= max_splits && splits * 2 * p.waves <= pairs) splits *= 2;
      kpw = ceil_div(pairs, splits * p.waves);
    };
    split_k();
    // activations in LDS when M <= 16, a wavefront has three or more pairs of K-blocks (two with more than 8
    // activation rows: N = K = 4096, M = 16: 7.2 -> 6.5 us, M = 1: 5.8 -> 5.9 us) and they fit beside the slabs.  A chunk has exactly the 4-row groups it needs (instantiated: 1, 2, 3, 4, 6, 8, 12, 16) when M <= 16,
    // whole 16-row groups otherwise.
    static const int kQ[] = {1, 2, 3, 4, 6, 8, 12, 16};
    auto round_q = [&](int need) { int q = 16; for (int i = 7; i >= 0; --i) if (kQ[i] >= need) q = kQ[i]; return q; };
    int q = round_q(p.q);
    auto place_activations = [&]() {
      p.xlds = p.tmx == 1 && kpw >= (M > 8 ? 2 : 3) && decode_lds_bytes_per_wave(q, p.waves, M, std::min<int64_t>(pairs, kpw * p.waves)) <= kDecodeLdsLimit;
      // Too large for LDS as a whole: two slots per wavefront, pair i + 1 copied while pair i is multiplied.  Only for
      // chunks with at least as many rows as there are activation rows (N = 7168, K = 16384, M = 16: 25.9 -> 22.9 us;
      // N = 4608, K = 7168: 11.0 -> 10.0; N = K = 8192: 17.9 -> 16.8; narrower chunks move more activation than weight
      // bytes and do better with fewer, taller chunks below: N = 1024, K = 8192, M = 16: 7.9 us there, 9.8 us here).
      // Where everything fits, the copies up front win: the same loop on N = 2112, K = 7168 takes 7.4 instead of 5.7 us.
      p.ring = !p.xlds && p.tmx == 1 && kpw >= (M > 8 ? 2 : 3) && ceil_div(N, chunks) >= M &&
               decode_lds_bytes_per_wave(q, p.waves, M, 2 * p.waves) <= kDecodeLdsLimit;
      if (p.ring) p.xlds = true;
    };
    place_activations();
    if (!p.xlds && p.tmx == 1 && M > 4 && N <= 64 * B) {
      // every block fetches all M activation rows of its K range per pair of K-blocks: chunks of fewer rows than
      // that move more activation than weight bytes (N = 2048, K = 1024, M = 16: 256 chunks of 8 rows 3.8 us,
      // 128 of 16 rows 3.5 us; N = 1024, K = 8192: 9.1 against 7.9 us); the K ranges of the taller chunks may fit LDS
      // (N = 1024, K = 8192, M = 16, 64 chunks in two ranges: 7.9 -> 6.9 us; N = 1280: 8.2 -> 7.4 us)
      deal_rows((M + 3) / 4 * 4);
      split_k();
      q = round_q(p.q);
      place_activations();
    }
    // Long K against narrow weights, 125 KB of activations or more (9 rows of K = 14336: 16.7 -> 14.0 us): every block reads the activations of its K range,
    // which at one range is as much as its weight rows or more.  Half the blocks with twice the rows (32 at most: taller
    // chunks take the slower four-group form) on half of K each halve the activation bytes per block, and the half
    // ranges may fit LDS.  us at M = 8 / 12 / 16, one range -> two: N = 2304, K = 16384: 15.6 / 14.7 / 17.6 -> 11.0 / 12.4 / 12.5;
    // N = 3584, K = 18944: 17.7 / 20.9 / 19.8 -> 16.0 / 16.7 / 16.7; M = 12 / 16: N = 4096, K = 14336: 16.4 / 16.9 -> 14.9 / 15.0;
    // N = 4096, K = 11008: 13.9 / 14.4 -> 12.7 / 12.9; M = 16: N = 3072, K = 8192: 10.3 -> 9.5.  Not below 128 KB (M = 8,
    // K = 14336: 12.4 -> 13.9; M = 12, N = 3072, K = 8192: 7.7 -> 9.5), not where the activations fit LDS at one range
    // (N = 2112, K = 7168, M = 16: 7.6 -> 8.0), not for taller chunks (N = 7168, K = 16384: 22.9 -> 27.5; N = 5120, K = 13824:
    // 16.7 -> 20.5).
    if (p.tmx == 1 && entries == 1 && M * KB >= 1000 && (!p.xlds || p.ring) && N <= 32 * (B / 2) && max_splits >= 2 && pairs >= 2 * 8) {
      deal_rows((M + 3) / 4 * 4, B / 2);
      p.n_chunks = (int)chunks;
      splits = 2;
      kpw = ceil_div(pairs, splits * p.waves);
      q = round_q(p.q);
      place_activations();
    }
    p.q = p.tmx == 1 ? q : 4 * p.rg;
  } else {
    // aim for ~8 wavefronts per CU on 256 CUs, each with at least one K-block
    const int64_t units = (int64_t)p.n_chunks * entries * KB;
    kpw = units / 2048;
    if (kpw < 1) kpw = 1;
    splits = ceil_div(KB, kpw * p.waves);
    if (splits < 1) splits = 1;
    if (splits > max_splits) splits = max_splits;
    kpw = ceil_div(KB, splits * p.waves);  // even out
    // a block with idle wavefronts wastes launch slots: fewer wavefronts when K is short
    if (splits == 1 && KB <= 4) { p.waves = 4; kpw = ceil_div(KB, 4); }
  }
  // Wide weights (five or more 16-row groups per compute unit, M <= 16): a wavefront per 16 rows walks all of K, four
  // wavefronts to a block that shares the activations through LDS; two or more such blocks fit a compute unit.
  // Measured against whole chunks shared by eight wavefronts: N = 24576, K = 1536: 12.3 -> 9.2 us; N = 32768,
  // K = 512: 6.5 -> 6.1 us; N = 28672, K = 4096: 26.5 -> 25 us; N = 16384, K = 2048 (four groups per unit): no gain.
  // With more than 16 pairs of K-blocks the walk of a single wavefront gets long and the shared chunks are as fast
  // (N = 32768, K = 8192: 51 us shared, 53-56 us here), so this form stops at K = 4096.
  // Up to 32 rows take the same form, with two 16-row images of the activations: against the 32-row chunks with the
  // activations in the register ring and the four-stage tile kernel, us at M = 17 / 24 / 32, before -> after:
  // N = 24576, K = 1536: 15.1 / 13.8 / 13.7 -> 10.5 / 11.3 / 12.3 (16 rows: 10.1); N = 49152, K = 1024: 20.4 / 21.3 / 22.6 ->
  // 12.5 / 13.3 / 17.4; N = 32768, K = 512: 8.4 / 8.5 / 8.7 -> 7.0 / 7.6 / 8.4.
  // Where two blocks of four wavefronts do not fit a compute unit but one of eight does, eight share the activations:
  // N = 20480, K = 3072, M = 24 / 32: 23.2 / 21.3 -> 15.5 / 16.5; N = 28672, K = 4096, M = 16 / 17 / 24: 28.5 / 32.7 / 33.4 ->
  // 27.4 / 26.6 / 27.3; N = 32768, K = 2048, M = 32: 20.8 -> 15.6.
  // With 17 to 32 rows the alternatives are weaker and four groups per compute unit suffice while K is short (N = 16384,
  // K = 1024, M = 17 / 24 / 32: 10.9 / 10.8 / 10.7 -> 7.3 / 7.5 / 8.2 us; N = 18432: 11.2 / 11.1 / 10.8 -> 8.2 / 8.7 / 9.3; K = 2048:
  // 11.8 / 12.0 / 12.6 -> 11.2 / 11.6 / 12.0; three groups, N = 12288, K = 1536: 9.3 -> 9.4, and N = 14336, K = 4096: 17.8 -> 19.7).
  // Up to 16 rows, K <= 2048: from the first row past 64 per compute unit on, where the shared chunks need a second round
  // of blocks (N = 18432, K = 1024, M = 1 / 16: 8.0 / 9.1 -> 7.1 / 7.9 us; N = 17408, K = 1536: 9.2 / 10.3 -> 8.7 / 9.6; at exactly
  // 64 rows, N = 16384, K = 2048: 8.7 -> 9.9, so not there).
  const int64_t groups = ceil_div(N, 16) * entries, cus = cu_count();
  const bool enough = KB > 16 ? groups >= 5 * cus : (p.tmx >= 2 ? groups >= 4 * cus : groups > 4 * cus);
  // 33 to 48 rows (four 16-row images): against the staged-activation and tile kernels it wins from twelve K-blocks on, and
  // from eight against weights of up to five groups per compute unit at up to 40 rows; us at M = 33 / 40 / 48, before -> after:
  // N = 49152, K = 2048: 38.8 / 38.6 / 39.0 -> 29.2 / 29.9 / 32.1; N = 24576, K = 1536: 15.0 / 14.2 / 14.2 -> 12.8 / 13.2 / 14.1;
  // N = 16384, K = 1024: 10.9 / 10.9 -> 8.9 / 9.4.  Not with fewer K-blocks or more rows (N = 32768, K = 512: 8.1 -> 8.9;
  // N = 49152, K = 1024, M = 48: 19.0 -> 20.5; 64 rows: 14.4 -> 15.9 and 10.8 -> 12.1 on the second and third shape above).
  const bool rows_ok = p.tmx <= 2 || (p.tmx == 4 && ((KB >= 12 && M <= 48) || (KB >= 8 && groups <= 5 * cus && M <= 40)));
  const bool own_shape = rows_ok && KB >= 2 && KB <= 32 && enough;
  const int own_waves = !own_shape ? 0 : decode_lds_bytes(4, 4, M, KB) <= kDecodeLdsLimit / 2 ? 4
                        : decode_lds_bytes(4, 8, M, KB) <= kDecodeLdsLimit ? 8 : 0;
  p.own = own_waves != 0;
  if (p.own) {
    p.staged = true; p.xlds = true; p.ring = false; p.q = 4; p.rg = 1; p.waves = own_waves; splits = 1; kpw = (KB + 1) / 2;
    p.n_chunks = (int)ceil_div(N, 16);
  }
  p.kpw = (int)kpw;
  p.splits = (int)splits;
  p.workspace_bytes = splits > 1
      ? (size_t)FG_WORKSPACE_COUNTER_BYTES + (size_t)p.n_chunks * splits * 16 * p.tmx * 16 * p.rg * sizeof(float)
      : 0;
  p.use = true;
  return p;
}

int launch_small_m(const GemmArgs& g, int mode, const SmallMPlan& plan, void* workspace, size_t workspace_bytes,
                   hipStream_t stream) {
  SmallArgs sa;
  sa.g = g;
  sa.kpw = plan.kpw;
  sa.splits = plan.splits;
  sa.n_chunks = plan.n_chunks;
  sa.rows_lo = (int)(g.N / plan.n_chunks);
  sa.rows_rem = (int)(g.N % plan.n_chunks);
  sa.x_lds_stride = plan.xlds ? x_lds_stride_for(std::min<int64_t>(g.KB, (int64_t)plan.kpw * plan.waves * 2)) : 0;
  sa.m_recip = (int)(65535 / g.M + 1);
  sa.pw_pairs = plan.ring ? 2 * plan.waves : (int)std::min<int64_t>((g.KB + 1) / 2, (int64_t)plan.kpw * plan.waves);
  sa.partials = nullptr;
  sa.counters = nullptr;
  sa.partials_per_entry = 0;
  if (plan.splits > 1) {
    const size_t entries = g.batch > 1 ? (size_t)g.batch : 1;
    const size_t per_entry = plan.workspace_bytes - FG_WORKSPACE_COUNTER_BYTES;
    const size_t need = FG_WORKSPACE_COUNTER_BYTES + entries * per_entry;
    sa.partials_per_entry = (int64_t)(per_entry / sizeof(float));
    if (entries * (size_t)plan.n_chunks * sizeof(unsigned int) > FG_WORKSPACE_COUNTER_BYTES)
      FG_FAIL(FG_ERR_WORKSPACE, "fp8 gemm (small M): %zu batch entries of %d chunks do not fit the counter area", entries, plan.n_chunks);
    if (!workspace || workspace_bytes < need)
      FG_FAIL(FG_ERR_WORKSPACE, "fp8 gemm (small M): workspace of %zu bytes needed, %zu given", need,
              workspace_bytes);
    if ((uintptr_t)workspace % 16 != 0) FG_FAIL(FG_ERR_INVALID_ARG, "fp8 gemm (small M): workspace must be 16-byte aligned");
    sa.counters = reinterpret_cast<unsigned int*>(workspace);
    sa.partials = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + FG_WORKSPACE_COUNTER_BYTES);
  }
  if (plan.staged) {
    // the staged kernels address with 32-bit lane offsets from uniform bases
    const uint64_t lim = 1ull << 32;
    if (g.ldw <= 0 || g.ldx <= 0 || g.xs_rs < 0 || g.xs_cs < 0 || (uint64_t)g.ldw * 64 + (uint64_t)g.K >= lim ||
        (uint64_t)g.ldx * 64 + (uint64_t)g.K >= lim || ((uint64_t)g.xs_rs * 64 + (uint64_t)g.xs_cs * g.KB) * 4 >= lim ||
        g.ws_rs < 0 || g.ws_cs < 0 || ((uint64_t)g.ws_rs + (uint64_t)g.ws_cs * g.KB) * 4 >= lim)
      FG_FAIL(FG_ERR_UNSUPPORTED, "fp8 gemm (small M): row strides of %lld / %lld bytes are beyond the kernel's 32-bit offsets",
              (long long)g.ldx, (long long)g.ldw);
    if (g.batch > 65535) FG_FAIL(FG_ERR_UNSUPPORTED, "fp8 gemm (small M): at most 65535 batch entries per launch, got %d", g.batch);
    if (plan.own && plan.tmx == 4)
      return plan.waves == 8 ? launch_transpose<4, 4, 1, 8, true, true>(sa, mode, stream) : launch_transpose<4, 4, 1, 4, true, true>(sa, mode, stream);
    if (plan.own && plan.waves == 8)
      return plan.tmx == 2 ? launch_transpose<2, 4, 1, 8, true, true>(sa, mode, stream) : launch_transpose<1, 4, 1, 8, true, true>(sa, mode, stream);
    if (plan.own) return plan.tmx == 2 ? launch_transpose<2, 4, 1, 4, true, true>(sa, mode, stream) : launch_transpose<1, 4, 1, 4, true, true>(sa, mode, stream);
    if (plan.xlds && plan.ring) {
      switch (plan.q) {
        case 1: return launch_transpose<1, 1, 1, 8, true, false, true>(sa, mode, stream);
        case 2: return launch_transpose<1, 2, 1, 8, true, false, true>(sa, mode, stream);
        case 3: return launch_transpose<1, 3, 1, 8, true, false, true>(sa, mode, stream);
        case 4: return launch_transpose<1, 4, 1, 8, true, false, true>(sa, mode, stream);
        case 6: return launch_transpose<1, 6, 1, 8, true, false, true>(sa, mode, stream);
        case 8: return launch_transpose<1, 8, 1, 8, true, false, true>(sa, mode, stream);
        case 12: return launch_transpose<1, 12, 1, 8, true, false, true>(sa, mode, stream);
        default: return launch_transpose<1, 16, 1, 8, true, false, true>(sa, mode, stream);
      }
    }
    if (plan.xlds) {
      switch (plan.q) {
        case 1: return launch_transpose<1, 1, 1, 8, true>(sa, mode, stream);
        case 2: return launch_transpose<1, 2, 1, 8, true>(sa, mode, stream);
        case 3: return launch_transpose<1, 3, 1, 8, true>(sa, mode, stream);
        case 4: return launch_transpose<1, 4, 1, 8, true>(sa, mode, stream);
        case 6: return launch_transpose<1, 6, 1, 8, true>(sa, mode, stream);
        case 8: return launch_transpose<1, 8, 1, 8, true>(sa, mode, stream);
        case 12: return launch_transpose<1, 12, 1, 8, true>(sa, mode, stream);
        default: return launch_transpose<1, 16, 1, 8, true>(sa, mode, stream);
      }
    }
    if (plan.tmx == 1) {
      switch (plan.q) {
        case 1: return launch_transpose<1, 1, 4, 8, false>(sa, mode, stream);
        case 2: return launch_transpose<1, 2, 4, 8, false>(sa, mode, stream);
        case 3: return launch_transpose<1, 3, 4, 8, false>(sa, mode, stream);
        case 4: return launch_transpose<1, 4, 4, 8, false>(sa, mode, stream);
        case 6: return launch_transpose<1, 6, 3, 8, false>(sa, mode, stream);
        case 8: return launch_transpose<1, 8, 3, 8, false>(sa, mode, stream);
        case 12: return launch_transpose<1, 12, 2, 8, false>(sa, mode, stream);
        default: return launch_transpose<1, 16, 2, 8, false>(sa, mode, stream);
      }
    }
    if (plan.rg == 1) return launch_transpose<2, 4, 3, 8, false>(sa, mode, stream);
    if (plan.rg == 2) return launch_transpose<2, 8, 2, 8, false>(sa, mode, stream);
    return launch_transpose<2, 16, 2, 4, false>(sa, mode, stream);
  }
  if (plan.tmx == 1) return plan.waves == 8 ? launch_t<1, 8>(sa, mode, stream) : launch_t<1, 4>(sa, mode, stream);
  if (plan.tmx == 2) return plan.waves == 8 ? launch_t<2, 8>(sa, mode, stream) : launch_t<2, 4>(sa, mode, stream);
  return launch_t<4, 4>(sa, mode, stream);
}

}  // namespace fg
