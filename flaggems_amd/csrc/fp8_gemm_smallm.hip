// Small-M (decode) FP8 GEMM for gfx950: M <= 64 activation rows against an [N, K] weight that is read
// exactly once.  The kernel is bound by HBM bandwidth, so the design is about bytes in flight, not
// about the matrix core:
//
//  * Work unit = (64 weight rows) x (one 128-byte K-block).  A wavefront streams its units straight
//    from global memory into registers: lane l owns weight row (l & 15) of each of the four 16-row
//    groups and the K bytes [16g, 16g+16) and [64+16g, 64+16g+16), g = l >> 4 -- the MFMA operand
//    layout, so no LDS staging is needed; the tiny activation fragment is fetched the same way (it
//    stays in L2).  The next unit's loads are issued before the current unit is multiplied.
//  * A block of 4 or 8 wavefronts shares one 64-row output chunk; its wavefronts take interleaved
//    K-blocks (adjacent wavefronts read adjacent 128-byte pieces of the same rows) and add their
//    fp32 results in LDS.
//  * When N/64 chunks do not give enough blocks to cover the GPU, several blocks split K.  Each
//    writes an fp32 partial tile to the workspace; the block that arrives last (a counter per
//    chunk) adds the partials in split order -- a fixed order, so results do not depend on timing --
//    and resets the counter, so the workspace needs zeroing only once, when it is allocated.
//
// Arithmetic follows the tile kernel: per K-block products accumulated by the fp8 MFMA, multiplied by
// As[m, kb] * Bs[n / 128, kb] in fp32 (block mode) or accumulated unscaled and scaled per row and column
// at the end (row/column mode).

#include "fp8_gemm_common.h"

namespace fg {
namespace {

constexpr int kChunkRows = 64;  // weight rows per block
constexpr int kRowGroups = 4;   // 16-row MFMA groups per chunk

struct SmallArgs {
  GemmArgs g;
  int kpw, splits, n_chunks;
  float* partials;      // [n_chunks][splits][16 * TMX][64]
  unsigned int* counters;
  int64_t partials_per_entry;  // floats; a batch (g.batch > 1, entry = blockIdx.y) keeps one such array and n_chunks counters per entry
};

// blockIdx.y-th problem of a batch: operands, partial sums and counters of that entry
__device__ __forceinline__ void select_batch_entry(SmallArgs& a) {
  if (a.g.batch > 1) {  // uniform
    const int64_t z = blockIdx.y;
    a.g.X += z * a.g.x_batch_bytes;
    a.g.W += z * a.g.w_batch_bytes;
    a.g.C = reinterpret_cast<uint8_t*>(a.g.C) + z * a.g.c_batch_bytes;
    a.g.xs += z * a.g.xs_batch_stride;
    a.g.ws += z * a.g.ws_batch_stride;
    if (a.partials) a.partials += z * a.partials_per_entry;
    if (a.counters) a.counters += z * a.n_chunks;
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
        acc[r][t] = mfma_fp8_16x16x128(wf, xf, acc[r][t]);
      }
    }
  }
}

// Adds the wavefronts' accumulators in LDS and writes the chunk (or publishes a split-K partial tile and,
// in the block that arrives last, adds the partial tiles in split order).  `red` is [WAVES][16*TMX][64].
template <int TMX, int RG, int WAVES, int MODE>
__device__ __forceinline__ void finish_chunk(const SmallArgs& a, float* red, int* last_flag,
                                             const v4f (&acc)[RG][TMX], int chunk, int split) {
  constexpr int NT = WAVES * 64;
  constexpr int MROWS = 16 * TMX;
  constexpr int kChunkRows = 16 * RG;
  constexpr int kRowGroups = RG;
  constexpr int kOut = MROWS * kChunkRows;
  const GemmArgs& g = a.g;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lg = lane >> 4;
  const int n0 = chunk * kChunkRows;
  // lane holds m = t*16 + l16, n = r*16 + 4*lg + [0,4)
#pragma unroll
  for (int r = 0; r < kRowGroups; ++r)
#pragma unroll
    for (int t = 0; t < TMX; ++t)
      *reinterpret_cast<v4f*>(red + ((wave * MROWS + t * 16 + l16) * kChunkRows + r * 16 + lg * 4)) = acc[r][t];
  __syncthreads();

  if (a.splits == 1) {
    for (int i = tid; i < kOut; i += NT) {
      const int m = i / kChunkRows, nn = i % kChunkRows;
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) v += red[w * kOut + i];
      if (m < g.M && n0 + nn < g.N) store_output<MODE>(g, m, n0 + nn, v);
    }
    return;
  }

  float* const mine = a.partials + ((int64_t)chunk * a.splits + split) * kOut;
  for (int i = tid; i < kOut; i += NT) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) v += red[w * kOut + i];
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
      v += __hip_atomic_load(all + (int64_t)s * kOut + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (m < g.M && n0 + nn < g.N) store_output<MODE>(g, m, n0 + nn, v);
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
  select_batch_entry(a);
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

  finish_chunk<TMX, kRowGroups, WAVES, MODE>(a, &red[0][0][0], &last_flag, acc, chunk, split);
}

// ---------------------------------------------------------------------------------------------
// Transposing variant (M <= 32, K >= 1024).  Same decomposition, but the weight bytes are fetched in
// runs of 256 contiguous bytes per row (two K-blocks; 4 rows per wavefront load instruction) instead
// of the 64-byte pieces the MFMA operand layout dictates: measured on MI355X a pure load of a
// [7168, 16384] matrix reaches 5.8 TB/s with 256-byte runs against 5.0 TB/s with 64-byte pieces.  The
// loads land in registers (the register file holds far more bytes in flight than LDS could); when a
// pair of K-blocks has arrived the wavefront writes it to its private 16 KB LDS slab and reads it back
// in operand layout.  No barrier is involved before the final reduction: a wavefront's LDS operations
// execute in order.  Within a row the sixteen 16-byte chunks are permuted (physical chunk p holds
// logical chunk p ^ (row & 15)) so that both the writes (4 rows x 256 B) and the operand reads (16 rows
// 256 bytes apart) spread over all LDS banks.
// ---------------------------------------------------------------------------------------------
template <int TMX, int RG>
struct PairRegs {
  u32x4 w[4 * RG];             // load j: rows 4j..4j+3, lane -> row 4j + (l >> 4), bytes 16*(l & 15) of the pair
  u32x4 xlo[2][TMX], xhi[2][TMX];
  float xs[2][TMX];
  float ws[2];
};

// RG = 16-row groups per chunk (1, 2 or 4), DEPTH = K-block pairs in flight per wavefront.
template <int TMX, int RG, int DEPTH, int WAVES, int MODE>
__global__ __launch_bounds__(WAVES * 64) void fp8_gemm_transpose_kernel(SmallArgs a) {
  constexpr int kRows = 16 * RG;
  constexpr int kSlab = kRows * 256;  // one K-block pair of the chunk
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];  // WAVES slabs; later the reduction buffer
  __shared__ int last_flag;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  select_batch_entry(a);
  const int chunk = blockIdx.x % a.n_chunks;
  const int split = blockIdx.x / a.n_chunks;
  const int n0 = chunk * kRows;
  const int l16 = lane & 15, lg = lane >> 4;
  const GemmArgs& g = a.g;
  uint8_t* const slab = lds + wave * kSlab;

  const uint8_t* const w_base = g.W + (int64_t)n0 * g.ldw + l16 * 16;
  const int rows_valid = g.N - n0;
  uint32_t w_off[4 * RG];
#pragma unroll
  for (int j = 0; j < 4 * RG; ++j) {
    int r = 4 * j + lg;
    r = r < rows_valid ? r : rows_valid - 1;  // rows past the edge alias the last valid row; never stored
    w_off[j] = (uint32_t)r * (uint32_t)g.ldw;
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

  v4f acc[RG][TMX];
#pragma unroll
  for (int r = 0; r < RG; ++r)
#pragma unroll
    for (int t = 0; t < TMX; ++t) acc[r][t] = v4f{0.f, 0.f, 0.f, 0.f};

  const int pairs_total = (g.KB + 1) >> 1;
  const int per_split = a.kpw * WAVES;
  const int pair_end = min(pairs_total, (split + 1) * per_split);

  auto load_pair = [&](PairRegs<TMX, RG>& u, int pair) __attribute__((always_inline)) {
    const int kb = pair * 2;
    const bool two = kb + 1 < g.KB;  // an odd K-block count leaves a single block at the end
    const int64_t k = (int64_t)kb * 128;
    // lanes 8..15 of a row own the second K-block; when it does not exist they re-read the first
    const int64_t kw = k - ((!two && l16 >= 8) ? 128 : 0);
#pragma unroll
    for (int j = 0; j < 4 * RG; ++j)
      u.w[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(w_base + kw + w_off[j]));
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int kbb = kb + ((b == 1 && two) ? 1 : 0);
#pragma unroll
      for (int t = 0; t < TMX; ++t) {
        u.xlo[b][t] = *reinterpret_cast<const u32x4*>(xrow[t] + (int64_t)kbb * 128);
        u.xhi[b][t] = *reinterpret_cast<const u32x4*>(xrow[t] + (int64_t)kbb * 128 + 64);
        if (MODE == kModeBlock) u.xs[b][t] = xsrow[t][(int64_t)kbb * g.xs_cs];
      }
      if (MODE == kModeBlock) u.ws[b] = wsrow[(int64_t)kbb * g.ws_cs];
    }
  };

  auto multiply = [&](const PairRegs<TMX, RG>& u, int pair) __attribute__((always_inline)) {
    const bool two = pair * 2 + 1 < g.KB;
    // registers -> slab: row R = 4j + lg, logical chunk l16 goes to physical chunk l16 ^ (R & 15)
#pragma unroll
    for (int j = 0; j < 4 * RG; ++j) {
      const int R = 4 * j + lg;
      *reinterpret_cast<u32x4*>(slab + R * 256 + ((l16 ^ (R & 15)) << 4)) = u.w[j];
    }
    // slab -> operand fragments: lane owns row rg*16 + l16 and logical chunks b*8 + lg, b*8 + lg + 4
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      if (b == 1 && !two) break;
#pragma unroll
      for (int r = 0; r < RG; ++r) {
        const uint8_t* row = slab + (r * 16 + l16) * 256;
        const u32x4 lo = *reinterpret_cast<const u32x4*>(row + (((b * 8 + lg) ^ l16) << 4));
        const u32x4 hi = *reinterpret_cast<const u32x4*>(row + (((b * 8 + lg + 4) ^ l16) << 4));
        const v8i wf = join(lo, hi);
#pragma unroll
        for (int t = 0; t < TMX; ++t) {
          const v8i xf = join(u.xlo[b][t], u.xhi[b][t]);
          if (MODE == kModeBlock) {
            const float sc = u.xs[b][t] * u.ws[b];
            const v4f p = mfma_fp8_16x16x128(wf, xf, v4f{0.f, 0.f, 0.f, 0.f});
            acc[r][t][0] = __builtin_fmaf(p[0], sc, acc[r][t][0]);
            acc[r][t][1] = __builtin_fmaf(p[1], sc, acc[r][t][1]);
            acc[r][t][2] = __builtin_fmaf(p[2], sc, acc[r][t][2]);
            acc[r][t][3] = __builtin_fmaf(p[3], sc, acc[r][t][3]);
          } else {
            acc[r][t] = mfma_fp8_16x16x128(wf, xf, acc[r][t]);
          }
        }
      }
    }
  };

  // DEPTH register sets form a ring; the loop body is written out once per set so that the ring index
  // is static and nothing is copied between sets
  int pair = split * per_split + wave;
  PairRegs<TMX, RG> ring[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (pair + d * WAVES < pair_end) load_pair(ring[d], pair + d * WAVES);
  bool done = pair >= pair_end;
  while (!done) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (!done) {
        multiply(ring[d], pair);
        const int refill = pair + DEPTH * WAVES;
        if (refill < pair_end) load_pair(ring[d], refill);
        pair += WAVES;
        done = pair >= pair_end;
      }
    }
  }
  __syncthreads();  // the slabs are dead; their memory now holds the reduction buffer
  finish_chunk<TMX, RG, WAVES, MODE>(a, reinterpret_cast<float*>(lds), &last_flag, acc, chunk, split);
}

template <int TMX, int WAVES>
int launch_t(const SmallArgs& sa, int mode, hipStream_t stream) {
  const dim3 grid((uint32_t)(sa.n_chunks * sa.splits), (uint32_t)(sa.g.batch > 1 ? sa.g.batch : 1)), block(WAVES * 64);
  if (mode == kModeBlock) FG_LAUNCH((fp8_gemm_smallm_kernel<TMX, WAVES, kModeBlock>), grid, block, 0, stream, sa);
  else FG_LAUNCH((fp8_gemm_smallm_kernel<TMX, WAVES, kModeRowCol>), grid, block, 0, stream, sa);
  FG_CHECK_LAUNCH("fp8_gemm_smallm_kernel");
  return FG_OK;
}

template <int TMX, int RG, int DEPTH, int WAVES>
int launch_transpose(const SmallArgs& sa, int mode, hipStream_t stream) {
  // WAVES slabs of RG * 4 KB; the reduction buffer (WAVES * 16*TMX * 16*RG floats) reuses the same memory
  constexpr int kSlabs = WAVES * 16 * RG * 256;
  constexpr int kRed = WAVES * 16 * TMX * 16 * RG * 4;
  constexpr int kLds = kSlabs > kRed ? kSlabs : kRed;
  const dim3 grid((uint32_t)(sa.n_chunks * sa.splits), (uint32_t)(sa.g.batch > 1 ? sa.g.batch : 1)), block(WAVES * 64);
  auto kb = fp8_gemm_transpose_kernel<TMX, RG, DEPTH, WAVES, kModeBlock>;
  auto kr = fp8_gemm_transpose_kernel<TMX, RG, DEPTH, WAVES, kModeRowCol>;
  static PerDeviceFlags lds_limit_raised = {};  // per instantiation
  {
    const hipError_t e = raise_dynamic_lds_limit(lds_limit_raised, kLds, reinterpret_cast<const void*>(kb), reinterpret_cast<const void*>(kr));
    if (e != hipSuccess) FG_FAIL(FG_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", kLds, hipGetErrorString(e));
  }
  if (mode == kModeBlock) FG_LAUNCH(kb, grid, block, kLds, stream, sa);
  else FG_LAUNCH(kr, grid, block, kLds, stream, sa);
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
  p.staged = p.tmx <= 2 && KB >= 8;
  if (p.staged) {
    // Rows per chunk: the largest of 64 / 32 / 16 that still yields at least ~140 blocks, so that K is
    // split across blocks only for very narrow weights (a split costs a round trip of partial tiles
    // through memory: measured 6.1 us unsplit against 8.6 us split in two for N = 2112, K = 7168).
    p.rg = 4;
    while (p.rg > 1 && ceil_div(N, 16 * p.rg) * entries < 140) p.rg >>= 1;
    p.waves = (p.tmx == 2 && p.rg == 4) ? 4 : 8;
  } else {
    p.waves = p.tmx == 4 ? 4 : 8;  // LDS reduction buffer is 4 KB * tmx per wavefront
  }
  p.n_chunks = (int)ceil_div(N, 16 * p.rg);
  if (p.n_chunks > FG_WORKSPACE_COUNTER_BYTES / 4) return p;
  // partial tiles cost 2 * splits * 16*tmx * rows * 4 bytes per chunk against rows * K weight bytes: keep
  // them under a quarter of the weight traffic
  const int64_t max_splits = K / (32 * 16 * p.tmx) > 1 ? K / (32 * 16 * p.tmx) : 1;
  if (p.staged) {
    const int64_t pairs = (KB + 1) / 2;
    splits = 1;
    while (p.n_chunks * entries * splits < 100 && splits * 2 <= max_splits && splits * 2 * p.waves <= pairs) splits *= 2;
    kpw = ceil_div(pairs, splits * p.waves);
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
    if (plan.tmx == 1) {
      if (plan.rg == 1) return launch_transpose<1, 1, 4, 8>(sa, mode, stream);
      if (plan.rg == 2) return launch_transpose<1, 2, 3, 8>(sa, mode, stream);
      return launch_transpose<1, 4, 2, 8>(sa, mode, stream);
    }
    if (plan.rg == 1) return launch_transpose<2, 1, 3, 8>(sa, mode, stream);
    if (plan.rg == 2) return launch_transpose<2, 2, 2, 8>(sa, mode, stream);
    return launch_transpose<2, 4, 2, 4>(sa, mode, stream);
  }
  if (plan.tmx == 1) return plan.waves == 8 ? launch_t<1, 8>(sa, mode, stream) : launch_t<1, 4>(sa, mode, stream);
  if (plan.tmx == 2) return plan.waves == 8 ? launch_t<2, 8>(sa, mode, stream) : launch_t<2, 4>(sa, mode, stream);
  return launch_t<4, 4>(sa, mode, stream);
}

}  // namespace fg
