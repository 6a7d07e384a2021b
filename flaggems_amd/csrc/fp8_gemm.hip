// FP8 (OCP e4m3fn) GEMM kernels for gfx950: block-scaled (1x128 activation scales, 128x128 weight
// scales) and per-row x per-column scaled with optional bias.
//
// Operand roles.  The problem is C[m, n] = sum_k X[m, k] * W[n, k] with both operands K-contiguous
// ("NT").  The weight tile takes the MFMA A slot and the activation tile the B slot
// (v_mfma_f32_16x16x128_f8f6f4 computes D[i][j] += sum_k A[i][k] B[j][k] with i = weight row n,
// j = activation row m).  A lane then holds four consecutive n for a single m, so one fp32 scale
// value As[m, kb] * Bs[n / 128, kb] covers all four of its results and the four results form one
// 8-byte bf16 store.
//
// Data path.  Tiles of BN x 128 weight bytes and BM x 128 activation bytes per K-block are staged in
// LDS, double buffered.  When rows are 16-byte aligned and K % 128 == 0 the tiles go from global
// memory straight into LDS (global_load_lds_dwordx4, 1 KB per wavefront instruction); otherwise a
// guarded register-staged loader zero-fills the K tail.  Tiles sit in LDS in fragment order (see
// the loaders below) so that every MFMA operand read is a lane-linear ds_read_b128.  In block-scaled mode every K-block's MFMA result is multiplied by its fp32
// scale and added to the running fp32 accumulator (4 VALU FMAs per MFMA); in row/column mode the
// MFMA accumulates directly and the scales are applied once in the epilogue.

#include "fp8_gemm_common.h"

#include <mutex>

namespace fg {
namespace {

// Map the hardware block id to a tile so that (a) the blocks one XCD receives (ids congruent mod 8)
// form a contiguous run of tiles and (b) a run walks GROUP_M tile rows before moving along N, which
// keeps the 32 tiles resident on an XCD inside a compact patch that shares operand panels in its L2.
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  const int xcd = bid & 7, local = bid >> 3;
  const int base = total >> 3, rem = total & 7;
  const int sid = xcd * base + (xcd < rem ? xcd : rem) + local;
  constexpr int GROUP_M = 4;
  const int per_group = GROUP_M * tiles_n;
  const int g = sid / per_group;
  const int first_m = g * GROUP_M;
  const int gm = (tiles_m - first_m < GROUP_M) ? tiles_m - first_m : GROUP_M;
  const int r = sid - g * per_group;
  tm = first_m + r % gm;
  tn = r / gm;
}

// ---------------------------------------------------------------------------------------------
// LDS image of a tile.  A tile is ROWS rows of one 128-byte K-block, row-major, with the eight
// 16-byte chunks of row R permuted: physical chunk p holds logical chunk p ^ (R & 7).  One
// global_load_lds_dwordx4 wavefront instruction fills 8 consecutive rows (1 KB, lane l writes byte
// l*16) and fetches 8 whole 128-byte lines.  Lane l of an MFMA operand fragment owns row (l & 15) and
// the logical chunks g and g+4 (g = l >> 4), i.e. K bytes [16g, 16g+16) and [64+16g, 64+16g+16); the K
// order inside a fragment therefore differs from memory order, identically for both operands, which
// leaves the dot product unchanged.  Both 16-byte reads of a fragment are bank-conflict free with this
// permutation (measured 218 B/clk/CU; 117 B/clk/CU when a lane reads the adjacent chunks 2g and 2g+1).
// ---------------------------------------------------------------------------------------------
template <int ROWS, int NTHREADS>
struct DirectTile {
  static constexpr int kWaves = NTHREADS / 64;
  static constexpr int kSlabs = ROWS / 8;  // 1 KB each
  static constexpr int kPerWave = kSlabs / kWaves;
  static_assert(kSlabs % kWaves == 0, "tile slabs must split evenly over the wavefronts");
  uint32_t off[kPerWave];  // byte offset of this lane's 16 bytes from the tile's first row, K-block 0

  // rows past the edge re-read the last valid row (their results are never stored)
  __device__ __forceinline__ void init(int64_t ld, int rows_valid, int wave, int lane) {
#pragma unroll
    for (int j = 0; j < kPerWave; ++j) {
      const int slab = wave + j * kWaves;
      const int r = slab * 8 + (lane >> 3);
      const int rc = r < rows_valid ? r : rows_valid - 1;
      off[j] = (uint32_t)rc * (uint32_t)ld + (uint32_t)(((lane & 7) ^ (r & 7)) << 4);
    }
  }
  // `base` is wave-uniform: first row of the tile, first byte of the K-block
  __device__ __forceinline__ void issue_one(const uint8_t* __restrict__ base, uint8_t* lds_tile, int wave, int j) const {
    const int slab = wave + j * kWaves;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base + off[j]),
                                     (__attribute__((address_space(3))) void*)(lds_tile + slab * 1024), 16, 0, 0);
  }
  __device__ __forceinline__ void issue(const uint8_t* __restrict__ base, uint8_t* lds_tile, int wave) const {
#pragma unroll
    for (int j = 0; j < kPerWave; ++j) issue_one(base, lds_tile, wave, j);
  }
};

template <int ROWS, int NTHREADS>
struct StagedTile {
  static constexpr int kChunks = ROWS * 8 / NTHREADS;
  static_assert(ROWS * 8 % NTHREADS == 0, "tile chunks must split evenly over the threads");
  u32x4 v[kChunks];

  // Loads with row and K guards; bytes past K are zero.  `aligned16` selects 16-byte loads.
  __device__ __forceinline__ void load(const uint8_t* __restrict__ g, int64_t ld, int row0, int row_max, int k0,
                                       int K, bool aligned16, int tid) {
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
      const int i = tid + j * NTHREADS;  // 16-byte chunk of the LDS image
      const int r = i >> 3;
      int gr = row0 + r;
      gr = gr < row_max ? gr : row_max;
      const int k = k0 + (((i & 7) ^ (r & 7)) << 4);
      const uint8_t* src = g + (int64_t)gr * ld + k;
      u32x4 t = {0u, 0u, 0u, 0u};
      if (aligned16 && k + 16 <= K) {
        t = *reinterpret_cast<const u32x4*>(src);
      } else if (k < K) {
        uint32_t w[4] = {0u, 0u, 0u, 0u};
        const int nb = (K - k < 16) ? K - k : 16;
        for (int b = 0; b < nb; ++b) w[b >> 2] |= (uint32_t)src[b] << (8 * (b & 3));
        t = u32x4{w[0], w[1], w[2], w[3]};
      }
      v[j] = t;
    }
  }
  __device__ __forceinline__ void store(uint8_t* lds_tile, int tid) const {
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
      const int i = tid + j * NTHREADS;
      *reinterpret_cast<u32x4*>(lds_tile + i * 16) = v[j];
    }
  }
};

// MFMA operand fragment of the 16-row group `rg` for this lane; `lane_off` = fragment_lane_offset(lane)
__device__ __forceinline__ int fragment_lane_offset(int lane) {
  const int r = lane & 15, g = lane >> 4;
  return r * 128 + ((g ^ (r & 7)) << 4);
}
__device__ __forceinline__ v8i read_fragment(const uint8_t* lds_tile, int rg, int lane_off) {
  // row group rg starts at rg*2048 and (16*rg) & 7 == 0, so the permutation depends on the lane only
  const u32x4 lo = *reinterpret_cast<const u32x4*>(lds_tile + rg * 2048 + lane_off);
  const u32x4 hi = *reinterpret_cast<const u32x4*>(lds_tile + rg * 2048 + (lane_off ^ 64));
  v8i f;
  f[0] = (int)lo.x; f[1] = (int)lo.y; f[2] = (int)lo.z; f[3] = (int)lo.w;
  f[4] = (int)hi.x; f[5] = (int)hi.y; f[6] = (int)hi.z; f[7] = (int)hi.w;
  return f;
}


// One K-block partial product with a zero accumulator input, result in architectural VGPRs.
__device__ __forceinline__ v4f mfma_fp8_block_partial(v8i a, v8i b) {
  v4f p = {};
  asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=&v"(p) : "v"(a), "v"(b));
  return p;
}

// acc += p * s.  `p` was written by the MFMA issued one step earlier (an 8-pass instruction): between
// that MFMA and these reads lie the previous step's four FMAs, one more MFMA and the s_nop below, which
// covers the 11 wait states gfx950 requires between an 8-pass matrix write and a VALU read of it.
#ifndef FG_MFMA_READ_NOPS
#define FG_MFMA_READ_NOPS 5
#endif
#define FG_STR2(x) #x
#define FG_STR(x) FG_STR2(x)
__device__ __forceinline__ void scale_accumulate(v4f& acc, const v4f& p, float s) {
  float a0 = acc[0], a1 = acc[1], a2 = acc[2], a3 = acc[3];
  asm volatile("s_nop " FG_STR(FG_MFMA_READ_NOPS) "\n\t"
               "v_fmac_f32 %0, %4, %8\n\t"
               "v_fmac_f32 %1, %5, %8\n\t"
               "v_fmac_f32 %2, %6, %8\n\t"
               "v_fmac_f32 %3, %7, %8"
               : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3)
               : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(s));
  acc[0] = a0; acc[1] = a1; acc[2] = a2; acc[3] = a3;
}

// Global -> LDS copies the compiler does not see (it would otherwise order every later LDS read behind them):
// 16 bytes per lane to lds_addr + 16 * lane, or 4 bytes per lane to lds_addr + 4 * lane.  `base` and `lds_addr`
// are wave-uniform; the copy counts in vmcnt and has landed in LDS when the counter says so.
__device__ __forceinline__ void copy_to_lds_16(uint32_t byte_off, const void* base, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\t"
               "s_nop 0\n\t"
               "global_load_lds_dwordx4 %0, %1"
               :
               : "v"(byte_off), "s"(base), "s"(lds_addr)
               : "memory", "m0");
}
__device__ __forceinline__ void copy_to_lds_4(uint32_t byte_off, const void* base, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\t"
               "s_nop 0\n\t"
               "global_load_lds_dword %0, %1"
               :
               : "v"(byte_off), "s"(base), "s"(lds_addr)
               : "memory", "m0");
}
template <int PENDING>
__device__ __forceinline__ void wait_vmem_at_most() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(PENDING) : "memory");
}

// NST: LDS stages.  2: the next K-block is loaded while the current one is multiplied.  More: NST - 1 K-blocks
// are in flight while one is multiplied (see "deep pipeline" in the kernel).
template <int BM, int BN, int WM, int WN, int NST = 2>
struct TileCfg {
  static constexpr int kThreads = WM * WN * 64;
  static constexpr int kWaveM = BM / WM, kWaveN = BN / WN;
  static constexpr int TM = kWaveM / 16, TN = kWaveN / 16;
  static constexpr int kStageBytes = (BM + BN) * 128;
  // activation scales of a stage: one per row (two stages), or one per thread (deep pipeline: every thread copies one)
  static constexpr int kScaleBytes = NST == 2 ? 2 * BM * 4 : NST * kThreads * 4;
  static constexpr int kLdsBytes = NST * kStageBytes + kScaleBytes;
  static_assert(BM <= kThreads, "one thread per activation row stages the row scales");
  static_assert(kWaveN <= 128 && 128 % kWaveN == 0, "a wavefront's N extent must stay inside one 128-wide scale block");
};

// ---------------------------------------------------------------------------------------------
// Main kernel
// ---------------------------------------------------------------------------------------------
// SPLIT: the grid is tiles x a.splits (times the batch in blockIdx.y, every entry with partial sums and counters of
// its own) and a block computes a range of K-blocks of its tile.  Every wavefront
// publishes its fp32 sums in the workspace and counts itself in (one counter per tile and wavefront position);
// the one that arrives last adds the sums of all splits in split order -- the same order whoever comes last --
// and runs the epilogue.  For problems with few tiles, which would leave most of the GPU idle while every
// K-block of a tile costs a full load latency.
template <int BM, int BN, int WM, int WN, int MODE, bool DIRECT, bool SPLIT = false, int NST = 2>
__global__ __launch_bounds__(WM* WN * 64) void fp8_gemm_kernel(GemmArgs a) {
  using Cfg = TileCfg<BM, BN, WM, WN, NST>;
  static_assert(NST == 2 || (DIRECT && NST >= 3 && NST <= 5), "deep pipeline: direct loads, 3..5 stages");
  if (a.batch > 1) {  // uniform: this workgroup's entry of the batch
    const int64_t z = blockIdx.y;
    a.X += z * a.x_batch_bytes;
    a.W += z * a.w_batch_bytes;
    a.C = reinterpret_cast<uint8_t*>(a.C) + z * a.c_batch_bytes;
    a.xs += z * a.xs_batch_stride;
    a.ws += z * a.ws_batch_stride;
    if (SPLIT && a.split_partials != nullptr) {
      a.split_partials += z * a.split_partials_per_entry;
      a.split_counters += z * (int64_t)(a.tiles_m * a.tiles_n * (Cfg::kThreads / 64));
    }
  }
  constexpr int NT = Cfg::kThreads;
  constexpr int TM = Cfg::TM, TN = Cfg::TN;
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  auto lds_w = [&](int stage) -> uint8_t* { return lds + stage * Cfg::kStageBytes; };
  auto lds_x = [&](int stage) -> uint8_t* { return lds + stage * Cfg::kStageBytes + BN * 128; };
  float* const lds_xs = reinterpret_cast<float*>(lds + NST * Cfg::kStageBytes);  // [2][BM], or [NST][NT]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave % WM, wave_n = wave / WM;

  int tile_id = (int)blockIdx.x, split = 0;
  if (SPLIT) {
    const int n_tiles = a.tiles_m * a.tiles_n;
    split = (int)blockIdx.x / n_tiles;
    tile_id = (int)blockIdx.x - split * n_tiles;
  }
  const int kb_begin = SPLIT ? split * a.kb_per_split : 0;
  const int kb_end = SPLIT ? (kb_begin + a.kb_per_split < a.KB ? kb_begin + a.kb_per_split : a.KB) : a.KB;
  int tile_m, tile_n;
  tile_of_block(tile_id, a.tiles_m, a.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int wm0 = wave_m * Cfg::kWaveM, wn0 = wave_n * Cfg::kWaveN;
  const int l16 = lane & 15, lg = lane >> 4;
  const int frag_off = fragment_lane_offset(lane);

  v4f acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  const bool aligned16 = ((a.ldx | a.ldw) % 16 == 0) && (((uintptr_t)a.X | (uintptr_t)a.W) % 16 == 0);
  StagedTile<BN, NT> st_w;
  StagedTile<BM, NT> st_x;
  DirectTile<BN, NT> dt_w;
  DirectTile<BM, NT> dt_x;
  (void)st_w; (void)st_x; (void)aligned16;
  // wave-uniform tile origins; a tile spans at most 256 rows, so lane offsets fit 32 bits (host checks ld)
  const uint8_t* const w_base = a.W + (int64_t)n0 * a.ldw;
  const uint8_t* const x_base = a.X + (int64_t)m0 * a.ldx;
  if (DIRECT) {
    dt_w.init(a.ldw, a.N - n0, wave, lane);
    dt_x.init(a.ldx, a.M - m0, wave, lane);
  }

  // activation-scale staging: thread t < BM owns row m0 + t
  const int xs_row = (m0 + tid < a.M) ? m0 + tid : a.M - 1;
  const float* xs_ptr = a.xs + (int64_t)xs_row * a.xs_rs;
  // weight-scale row of this wavefront's N range (one 128-wide block)
  const int nb_last = (a.N - 1) >> 7;
  const int wn_blk = ((n0 + wn0) >> 7) < nb_last ? ((n0 + wn0) >> 7) : nb_last;
  const float* ws_ptr = a.ws + (int64_t)wn_blk * a.ws_rs;

  if constexpr (NST > 2) {
    // ---- deep pipeline.  NST - 1 K-blocks are on their way into LDS while one is multiplied, so a K-block costs
    // 1 / (NST - 1) of a load latency instead of a whole one (a block that owns a compute unit alone -- few tiles,
    // K split over blocks -- is otherwise bound by exactly that latency).  Per K-block a wavefront issues
    // kPerStage copies in a fixed order (its thread's activation scale, then its slabs of the two tiles); vmcnt
    // retires them in order, so "at most p * kPerStage pending" means that all but the youngest p stages have
    // landed.  One barrier per K-block: behind it every wavefront's share of the stage is in LDS and nobody reads
    // the slot that the stage issued next overwrites.
    // (Measured and not kept: reading the fragments of K-block kb + 1 into a second register set under the MFMAs of
    // K-block kb.  With one wavefront per SIMD everything it issues is serial anyway; 3-8 % slower.)
    constexpr int kLoadsW = DirectTile<BN, NT>::kPerWave, kLoadsX = DirectTile<BM, NT>::kPerWave;
    constexpr int kPerStage = kLoadsW + kLoadsX + (MODE == kModeBlock ? 1 : 0);
    static_assert((NST - 2) * kPerStage <= 63, "vmcnt holds 6 bits");
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    const uint32_t lds_scales = lds_base + NST * Cfg::kStageBytes;
    // this thread's activation row (threads past the tile copy the last row's scale; nobody reads it)
    int xs_rel = tid < BM ? tid : BM - 1;
    xs_rel = (m0 + xs_rel < a.M) ? xs_rel : a.M - 1 - m0;
    const uint32_t xs_off = (uint32_t)xs_rel * (uint32_t)a.xs_rs * 4u;  // the host checks that 256 rows of scales fit 32 bits
    const float* const xs_tile = MODE == kModeBlock ? a.xs + (int64_t)m0 * a.xs_rs : nullptr;
    auto issue_scale = [&](int kb_load, int slot) __attribute__((always_inline)) {
      if (MODE != kModeBlock) return;
      copy_to_lds_4(xs_off, uniform_ptr(xs_tile + (int64_t)kb_load * a.xs_cs), lds_scales + (uint32_t)((slot * NT + wave * 64) * 4));
    };
    auto issue_tile_part = [&](int kb_load, int slot, int q) __attribute__((always_inline)) {
      if (q < kLoadsW) {
        const int slab = wave + q * (NT / 64);
        copy_to_lds_16(dt_w.off[q], uniform_ptr(w_base + (int64_t)kb_load * 128), lds_base + (uint32_t)(slot * Cfg::kStageBytes + slab * 1024));
      } else {
        const int slab = wave + (q - kLoadsW) * (NT / 64);
        copy_to_lds_16(dt_x.off[q - kLoadsW], uniform_ptr(x_base + (int64_t)kb_load * 128),
                       lds_base + (uint32_t)(slot * Cfg::kStageBytes + BN * 128 + slab * 1024));
      }
    };
    // (read through the constant address space: next to assembly that clobbers memory the compiler would otherwise
    // use a vector load, and its wait for that load would wait for every copy in flight)
    auto weight_scale = [&](int kb_) __attribute__((always_inline)) -> float {
      return *(const __attribute__((address_space(4))) float*)(ws_ptr + (int64_t)kb_ * a.ws_cs);
    };
    float ws_pend = 1.f, ws_cur = 1.f;
    for (int st = 0; st < NST - 1; ++st) {
      if (kb_begin + st < kb_end) {
        issue_scale(kb_begin + st, st);
#pragma unroll
        for (int q = 0; q < kLoadsW + kLoadsX; ++q) issue_tile_part(kb_begin + st, st, q);
      }
    }
    if (MODE == kModeBlock && kb_begin < kb_end) ws_pend = weight_scale(kb_begin);
    int cur = 0, load_slot = NST - 1;
    for (int kb = kb_begin; kb < kb_end; ++kb) {
      const int rem = kb_end - 1 - kb;  // stages issued after this one that may still be on their way
      if (rem >= NST - 2) wait_vmem_at_most<(NST - 2) * kPerStage>();
      else if (NST > 3 && rem == 1) wait_vmem_at_most<kPerStage>();
      else if (NST > 4 && rem == 2) wait_vmem_at_most<2 * kPerStage>();
      else wait_vmem_at_most<0>();
      // (a bare barrier: __syncthreads() carries a fence for which the compiler waits for every copy in flight.
      // The LDS reads of the previous K-block have returned: their values were consumed by its MFMAs.)
      __builtin_amdgcn_s_barrier();
      const int kb_load = kb + NST - 1;
      const bool more = kb_load < kb_end;
      if (MODE == kModeBlock) {
        ws_cur = ws_pend;
        if (kb + 1 < kb_end) ws_pend = weight_scale(kb + 1);
      }
      if (more) issue_scale(kb_load, load_slot);
      const uint8_t* const tw = lds_w(cur) + (wn0 >> 4) * 2048;
      const uint8_t* const tx = lds_x(cur) + (wm0 >> 4) * 2048;
      v8i xf[TM];
      xf[0] = read_fragment(tx, 0, frag_off);
      v8i wf = read_fragment(tw, 0, frag_off);
#pragma unroll
      for (int j = 1; j < TM; ++j) xf[j] = read_fragment(tx, j, frag_off);
      constexpr int kLoadEvery = (TN * TM) / (kLoadsW + kLoadsX);
      static_assert(kLoadEvery >= 1, "more tile loads than MFMA steps");
      if (MODE == kModeBlock) {
        float sc[TM];
#pragma unroll
        for (int j = 0; j < TM; ++j) sc[j] = lds_xs[cur * NT + wm0 + j * 16 + l16] * ws_cur;
        v4f p_prev = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < TN; ++i) {
          v8i wf_next = wf;
          if (i + 1 < TN) wf_next = read_fragment(tw, i + 1, frag_off);
#pragma unroll
          for (int j = 0; j < TM; ++j) {
            const v4f p = mfma_fp8_block_partial(wf, xf[j]);
            if (i > 0 || j > 0) {
              const int pi = (j == 0) ? i - 1 : i, pj = (j == 0) ? TM - 1 : j - 1;
              scale_accumulate(acc[pi][pj], p_prev, sc[pj]);
            }
            p_prev = p;
            const int t = i * TM + j;
            if (t % kLoadEvery == 0 && t / kLoadEvery < kLoadsW + kLoadsX && more) issue_tile_part(kb_load, load_slot, t / kLoadEvery);
          }
          wf = wf_next;
        }
        scale_accumulate(acc[TN - 1][TM - 1], p_prev, sc[TM - 1]);
      } else {
#pragma unroll
        for (int i = 0; i < TN; ++i) {
          v8i wf_next = wf;
          if (i + 1 < TN) wf_next = read_fragment(tw, i + 1, frag_off);
#pragma unroll
          for (int j = 0; j < TM; ++j) {
            acc[i][j] = MODE == kModeRowColI8 ? mfma_i8_16x16x128(wf, xf[j], acc[i][j]) : mfma_fp8_16x16x128(wf, xf[j], acc[i][j]);
            const int t = i * TM + j;
            if (t % kLoadEvery == 0 && t / kLoadEvery < kLoadsW + kLoadsX && more) issue_tile_part(kb_load, load_slot, t / kLoadEvery);
          }
          wf = wf_next;
        }
      }
      cur = (cur + 1 == NST) ? 0 : cur + 1;
      load_slot = (load_slot + 1 == NST) ? 0 : load_slot + 1;
    }
  } else {
  // ---- prologue: stage 0
  if (kb_begin >= kb_end) {
    // K == 0 (or an empty range): nothing to stage, the accumulators stay zero
  } else if (DIRECT) {
    dt_w.issue(w_base + kb_begin * 128, lds_w(0), wave);
    dt_x.issue(x_base + kb_begin * 128, lds_x(0), wave);
  } else {
    st_w.load(a.W, a.ldw, n0, a.N - 1, kb_begin * 128, a.K, aligned16, tid);
    st_x.load(a.X, a.ldx, m0, a.M - 1, kb_begin * 128, a.K, aligned16, tid);
    st_w.store(lds_w(0), tid);
    st_x.store(lds_x(0), tid);
  }
  // Scales travel one K-block ahead of the tiles: every wait for them then falls right after the
  // tile-load wait at the top of an iteration, where they have been in flight for a whole iteration.
  // (A wait at the end of the iteration would also wait for the tile loads issued moments before.)
  float xs_pend = 0.f, ws_pend = 1.f, ws_cur = 1.f;
  if (MODE == kModeBlock && kb_begin < kb_end) {
    if (tid < BM) {
      lds_xs[tid] = xs_ptr[(int64_t)kb_begin * a.xs_cs];
      if (kb_begin + 1 < kb_end) xs_pend = xs_ptr[(int64_t)(kb_begin + 1) * a.xs_cs];
    }
    ws_pend = ws_ptr[(int64_t)kb_begin * a.ws_cs];
  }

  for (int kb = kb_begin; kb < kb_end; ++kb) {
    const int cur = (kb - kb_begin) & 1, nxt = cur ^ 1;
    if (DIRECT) wait_vmem_all();
    __syncthreads();

    const bool more = kb + 1 < kb_end;
    if (MODE == kModeBlock) {
      ws_cur = ws_pend;
      if (more) {
        if (tid < BM) {
          lds_xs[nxt * BM + tid] = xs_pend;  // scales of K-block kb+1, read after the next barrier
          if (kb + 2 < kb_end) xs_pend = xs_ptr[(int64_t)(kb + 2) * a.xs_cs];
        }
        ws_pend = ws_ptr[(int64_t)(kb + 1) * a.ws_cs];
      }
    }
    if (more) {
      const int k1 = (kb + 1) * 128;
      if (DIRECT) {
        // block-scaled mode spreads the tile loads over the MFMA steps below: issued as one burst
        // they fill the CU's address queue and every wavefront stalls in the issue for ~1-2k cycles
        if (MODE != kModeBlock) {
          dt_w.issue(w_base + k1, lds_w(nxt), wave);
          dt_x.issue(x_base + k1, lds_x(nxt), wave);
        }
      } else {
        st_w.load(a.W, a.ldw, n0, a.N - 1, k1, a.K, aligned16, tid);
        st_x.load(a.X, a.ldx, m0, a.M - 1, k1, a.K, aligned16, tid);
      }
    }

    // ---- compute on stage `cur`
    const uint8_t* const tw = lds_w(cur) + (wn0 >> 4) * 2048;
    const uint8_t* const tx = lds_x(cur) + (wm0 >> 4) * 2048;
    // LDS reads in the order the first MFMAs need them: all wavefronts leave the barrier together
    // and the reads of this phase queue up in the LDS, so the first operands should be at the front
    v8i xf[TM];
    xf[0] = read_fragment(tx, 0, frag_off);
    v8i wf_first = read_fragment(tw, 0, frag_off);
#pragma unroll
    for (int j = 1; j < TM; ++j) xf[j] = read_fragment(tx, j, frag_off);
    float sc[TM];
    if (MODE == kModeBlock) {
#pragma unroll
      for (int j = 0; j < TM; ++j) sc[j] = lds_xs[cur * BM + wm0 + j * 16 + l16] * ws_cur;
    }
    if (MODE == kModeBlock) {
      // Software pipeline with a pinned issue order: MFMA t, then the four scale-FMAs of MFMA t-1,
      // which execute while the matrix core works on t.  The steps are volatile asm statements
      // because the compiler otherwise clusters all MFMAs of the K-block, keeps every partial result
      // live and spills the accumulators.
      v8i wf = wf_first;
      constexpr int kLoadsW = DirectTile<BN, NT>::kPerWave, kLoadsX = DirectTile<BM, NT>::kPerWave;
      constexpr int kLoadEvery = (TN * TM) / (kLoadsW + kLoadsX);
      static_assert(kLoadEvery >= 1, "more tile loads than MFMA steps");
      const uint8_t* const w_next = w_base + (kb + 1) * 128;
      const uint8_t* const x_next = x_base + (kb + 1) * 128;
      v4f p_prev = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        v8i wf_next = wf;
        if (i + 1 < TN) wf_next = read_fragment(tw, i + 1, frag_off);
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          const v4f p = mfma_fp8_block_partial(wf, xf[j]);
          if (i > 0 || j > 0) {
            const int pi = (j == 0) ? i - 1 : i, pj = (j == 0) ? TM - 1 : j - 1;
            scale_accumulate(acc[pi][pj], p_prev, sc[pj]);
          }
          p_prev = p;
          if (DIRECT) {
            const int t = i * TM + j;
            if (t % kLoadEvery == 0 && t / kLoadEvery < kLoadsW + kLoadsX && more) {
              const int q = t / kLoadEvery;
              if (q < kLoadsW) dt_w.issue_one(w_next, lds_w(nxt), wave, q);
              else dt_x.issue_one(x_next, lds_x(nxt), wave, q - kLoadsW);
            }
          }
        }
        wf = wf_next;
      }
      scale_accumulate(acc[TN - 1][TM - 1], p_prev, sc[TM - 1]);
    } else {
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        const v8i wf = (i == 0) ? wf_first : read_fragment(tw, i, frag_off);
#pragma unroll
        for (int j = 0; j < TM; ++j)
          acc[i][j] = MODE == kModeRowColI8 ? mfma_i8_16x16x128(wf, xf[j], acc[i][j]) : mfma_fp8_16x16x128(wf, xf[j], acc[i][j]);
      }
    }

    if (more) {
      if (!DIRECT) {
        st_w.store(lds_w(nxt), tid);
        st_x.store(lds_x(nxt), tid);
      }
    }
  }

  }

  if (SPLIT && a.splits > 1) {
    // element (i, j) of thread tid lives at ((i * TM + j) * NT + tid) * 16 bytes of the (tile, split) slot
    constexpr int kSlotFloats = TN * TM * NT * 4;
    const uint32_t t_off = (uint32_t)tid * 16u;
    float* const mine = uniform_ptr(a.split_partials + ((size_t)tile_id * a.splits + split) * kSlotFloats);
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TM; ++j) store_x4_agent(mine + (i * TM + j) * NT * 4, t_off, acc[i][j]);
    wait_vmem_all();
    unsigned int* const cnt = a.split_counters + tile_id * (NT / 64) + wave;
    unsigned int prev = 0;
    if (lane == 0) prev = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    prev = (unsigned int)__builtin_amdgcn_readfirstlane((int)prev);
    if (prev != (unsigned int)(a.splits - 1)) return;
    for (int s = 0; s < a.splits; ++s) {
      const float* const src = uniform_ptr(a.split_partials + ((size_t)tile_id * a.splits + s) * kSlotFloats);
      v4f tmp[TN][TM];
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j) load_x4_agent(tmp[i][j], src + (i * TM + j) * NT * 4, t_off);
#pragma unroll
      for (int i = 0; i < TN; ++i)  // the values are operands of the wait, so no use can move above it
#pragma unroll
        for (int j = 0; j < TM; ++j) asm volatile("s_waitcnt vmcnt(0)" : "+v"(tmp[i][j]) : : "memory");
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          // plain assignment for the first split keeps "0 + x" out of the sum; int8 operands: int32 sums, added as such
          if (s == 0) acc[i][j] = tmp[i][j];
          else if (MODE == kModeRowColI8) acc[i][j] = __builtin_bit_cast(v4f, __builtin_bit_cast(v4i, acc[i][j]) + __builtin_bit_cast(v4i, tmp[i][j]));
          else acc[i][j] += tmp[i][j];
        }
    }
    if (lane == 0) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- epilogue: the lane holds m = ... + l16, n = ... + 4 * lg + [0, 4) of every MFMA tile
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    const int m = m0 + wm0 + j * 16 + l16;
    if (m >= a.M) continue;
#pragma unroll
    for (int i = 0; i < TN; ++i) store_output4<MODE>(a, m, n0 + wn0 + i * 16 + lg * 4, acc[i][j]);
  }
}

template <int BM, int BN, int WM, int WN, int MODE, bool DIRECT>
int launch_cfg(GemmArgs a, hipStream_t stream) {
  using Cfg = TileCfg<BM, BN, WM, WN>;
  a.tiles_m = (int)ceil_div(a.M, BM);
  a.tiles_n = (int)ceil_div(a.N, BN);
  auto kern = fp8_gemm_kernel<BM, BN, WM, WN, MODE, DIRECT>;
  static PerDeviceFlags lds_limit_raised = {};  // per instantiation
  {
    const hipError_t e = raise_dynamic_lds_limit(lds_limit_raised, Cfg::kLdsBytes, reinterpret_cast<const void*>(kern));
    if (e != hipSuccess) FG_FAIL(FG_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", Cfg::kLdsBytes, hipGetErrorString(e));
  }
  const int64_t blocks = (int64_t)a.tiles_m * a.tiles_n;
  if (blocks > 0x7FFFFFFF) FG_FAIL(FG_ERR_UNSUPPORTED, "fp8 gemm: too many tiles");
  if (a.batch > 65535) FG_FAIL(FG_ERR_UNSUPPORTED, "fp8 gemm: more than 65535 batch entries in one launch");
  FG_LAUNCH(kern, dim3((uint32_t)blocks, (uint32_t)(a.batch > 1 ? a.batch : 1)), dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, a);
  FG_CHECK_LAUNCH("fp8_gemm_kernel");
  return FG_OK;
}

// M > 32 with at most 128 tiles of 128 x 128 (256 when K <= 8192): K split over blocks so that more than one block per compute unit is
// resident (a K-block of one tile costs a full load latency, ~1.8 us; the loads of several blocks overlap).
// Measured against the persistent kernel (which has a quarter of the tiles, and stream-K): M = 256, N = 2112,
// K = 7168: 79 -> 31 us; M = 512, N = 4096, K = 4096: 50 -> 28 us; M = 512, N = 1024, K = 8192: 83 -> 26 us.
struct TileSplitPlan {
  bool use;
  int splits, kb_per_split;
  size_t workspace_bytes;
};
// 128 x 128 tiles for problems with few tiles: eight wavefronts (4 x 2, each 32 x 64) rather than four: two per SIMD
// overlap one's LDS reads with the other's MFMAs (measured 10-18 % faster than four on every shape of this path).
constexpr int kSplitTile = 128, kSplitWM = 4, kSplitWaves = kSplitWM * 2;
TileSplitPlan plan_tile_split(int64_t M, int64_t N, int64_t K) {
  TileSplitPlan p = {false, 1, 0, 0};
  if (M <= 32 || M > 1024 || K % 128 != 0) return p;
  const int64_t KB = K / 128;
  const int64_t tiles = ceil_div(M, kSplitTile) * ceil_div(N, kSplitTile);
  if (tiles * kSplitWaves * 4 > FG_WORKSPACE_COUNTER_BYTES) return p;
  // 129..256 tiles: one block per compute unit, which waits out every K-block's load; two blocks per tile help while
  // K is at most 8192 (measured M = 512: N = 6144, K = 4096: 54 -> 33 us; 4608 x 7168: 56 -> 44; 7168 x 2304: 35 -> 27;
  // M = 1024: 4096 x 4096: 51 -> 38; but 4096 x 14336: 85 -> 97, so long K stays with the persistent kernel)
  if (tiles > 256 || (tiles > 128 && KB > 64)) return p;
  // up to 64 rows the decode kernels are the alternative: they win unless K is long (measured: K = 7168 and
  // 16384 faster here, K = 1024 ... 2304 faster there)
  if (M <= 64 && KB < 32) return p;
  int64_t splits = (320 + tiles / 2) / tiles;  // ~1.25 blocks per compute unit
  if (tiles > 128) splits = 2;
  if (splits > KB / 4) splits = KB / 4;  // at least four K-blocks per block
  if (splits > 8) splits = 8;            // the wavefront that finishes a tile reads the splits one after another
  if (splits < 2) return p;
  p.kb_per_split = (int)ceil_div(KB, splits);
  p.splits = (int)ceil_div(KB, (int64_t)p.kb_per_split);
  p.workspace_bytes = FG_WORKSPACE_COUNTER_BYTES + (size_t)tiles * p.splits * kSplitTile * kSplitTile * sizeof(float);
  p.use = p.splits >= 2;
  return p;
}

template <int MODE>
int launch_tile_split(GemmArgs a, const TileSplitPlan& plan, void* workspace, hipStream_t stream) {
  using Cfg = TileCfg<kSplitTile, kSplitTile, kSplitWM, 2>;
  a.tiles_m = (int)ceil_div(a.M, kSplitTile);
  a.tiles_n = (int)ceil_div(a.N, kSplitTile);
  a.splits = plan.splits;
  a.kb_per_split = plan.kb_per_split;
  a.split_counters = reinterpret_cast<unsigned int*>(workspace);
  a.split_partials = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(workspace) + FG_WORKSPACE_COUNTER_BYTES);
  auto kern = fp8_gemm_kernel<kSplitTile, kSplitTile, kSplitWM, 2, MODE, true, true>;
  static PerDeviceFlags lds_limit_raised = {};
  {
    const hipError_t e = raise_dynamic_lds_limit(lds_limit_raised, Cfg::kLdsBytes, reinterpret_cast<const void*>(kern));
    if (e != hipSuccess) FG_FAIL(FG_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", Cfg::kLdsBytes, hipGetErrorString(e));
  }
  const int64_t blocks = (int64_t)a.tiles_m * a.tiles_n * a.splits;
  FG_LAUNCH(kern, dim3((uint32_t)blocks), dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, a);
  FG_CHECK_LAUNCH("fp8_gemm_kernel (K split)");
  return FG_OK;
}

// M >= 65 with at most one 128 x 128 tile per compute unit: the tile kernel with four LDS stages, one block
// per compute unit, K split over blocks while blocks are fewer than compute units.  With two stages a block that
// has a compute unit to itself pays a whole load latency per K-block.  The tile count decides, not M: tall
// problems against narrow weights (M = 2048, N = 512, K = 7168: 128 tiles) took 73 us in the persistent kernel, which
// has a quarter of the tiles and shares them along K, and take 22 us here; with more tiles than compute units a
// second round of this kernel loses to the persistent kernel (M = 1024, N = 4608, K = 7168, 288 tiles: 62 -> 79 us).
struct PipePlan {
  bool use;
  int splits, kb_per_split;
  size_t workspace_bytes;
};
constexpr int kPipeStages = 4;
// entries: equal problems launched together (blockIdx.y = entry): their tiles fill the compute units together, and
// workspace_bytes is what all of them need.
// Whether the staged-activation kernel's blocks run in two or more rounds with the last one under nine tenths full.
bool mid_m_partial_round(const MidMPlan& mid, int cus) {
  if (!mid.use) return false;
  const int64_t blocks = ceil_div((int64_t)mid.n_chunks, (int64_t)mid.waves) * mid.splits;
  const int64_t slots = (int64_t)cus * (mid.waves == 8 ? 1 : 2);  // four-wavefront blocks take half of LDS at most
  const int64_t rounds = ceil_div(blocks, slots);
  return rounds >= 2 && blocks * 10 < rounds * slots * 9;
}

PipePlan plan_pipe(int64_t M, int64_t N, int64_t K, int64_t xs_rs, int64_t entries = 1) {
  PipePlan p = {false, 1, 0, 0};
  if (entries < 1) entries = 1;
  if (M <= 16 || (M <= 32 && entries > 1) || K <= 0 || K % 128 != 0) return p;
  if (xs_rs < 0 || xs_rs >= (1 << 21)) return p;  // 256 rows of scales addressed with 32-bit byte offsets
  const int64_t KB = K / 128;
  const int64_t tiles = ceil_div(M, kSplitTile) * ceil_div(N, kSplitTile) * entries;
  const int cus = cu_count();
  if (tiles > cus || KB < 4) return p;
  if (tiles * kSplitWaves * 4 > FG_WORKSPACE_COUNTER_BYTES) return p;
  int64_t splits = cus / tiles;
  if (splits > KB / 5) splits = KB / 5;  // at least five K-blocks per block: a block starts with a full load latency
  if (splits > 8) splits = 8;            // the wavefront that finishes a tile reads the splits one after another
  if (splits < 1) splits = 1;
  // 129 to 160 tiles unsplit leave over a third of the compute units idle for the whole launch; with long K three ranges
  // (1.7 to 1.9 rounds of blocks) pay for their partial tiles: M = 128: N = 18432, K = 16384: 110 -> 91 us; K = 8192:
  // 58 -> 53 us; N = 20480, K = 8192: 58 -> 55 us; M = 256: N = K = 9216: 66 -> 52 us; N = 10240, K = 8192: 53 -> 49 us.  Not with
  // short K or more tiles (M = 128, N = 24576, K = 4096, 192 tiles: 35 -> 46 us; M = 256, N = 13312, K = 16384, 208 tiles:
  // 89 -> 116 us), and two, five or seven ranges lose everywhere.  (Equal runs of K-blocks dealt out over the compute
  // units whatever the tile borders -- every block then writes up to two partial tiles and the blocks of a tile run at
  // different places in K -- were built and measured on 17 weight shapes x M = 128 / 256 / 512: faster on three of
  // the 51 cases by 12-16 %, slower by up to 2x where several row tiles share a weight block, 5-45 % slower where K is short.)
  if (splits == 1 && entries == 1 && M > 64 && tiles * 2 > cus && tiles * 16 <= (int64_t)cus * 10 && KB >= 64) splits = 3;
  p.kb_per_split = (int)ceil_div(KB, splits);
  p.splits = (int)ceil_div(KB, (int64_t)p.kb_per_split);
  // Long K loops stay with the persistent kernel, whose 256 x 256 tiles need half the LDS reads per MFMA (measured
  // with up to 128 K-blocks per block allowed here: M = 1024, N = 4096, K = 14336: 74 -> 82 us; with up to 64: M = 512,
  // same weights: 53 -> 45 us; N = 7168, K = 16384 at M = 256: 59 -> 50 us).
  if (p.kb_per_split > 64) return p;
  // 33..64 rows: half of every tile is padding, and so is half of every partial tile a split writes; the
  // staged-activation kernel is the alternative.  This kernel wins while K is split in two at most over ranges of
  // eight K-blocks or more (measured at M = 64: N = 28672, K = 4096, 224 tiles unsplit: 46 -> 32 us; N = 24576, K = 1536:
  // 16.2 -> 14.6 us; a batch of 16 x [1024, 7168], 128 tiles in two ranges, 48 rows: 41 -> 34 us; but N = 32768, K = 512,
  // four K-blocks: 8.5 -> 9.8 us; N = 4096, K = 14336 in eight ranges: 23 -> 25 us; N = 4608, K = 7168 in seven: 17 -> 20 us;
  // a batch of 8 x [1024, 4096] in four: 16 -> 20 us)
  // -- or while that kernel, one block of eight wavefronts per compute unit at these sizes, would run a second round
  // of blocks that fills under nine tenths of the compute units (M = 48: N = 10240, K = 8192, 320 blocks: 38 -> 26 us;
  // N = 7168, K = 8192, 280 blocks: 32.5 -> 23 us; N = 5120, K = 13824: 36 -> 25 us; N = 9216, K = 9216: 39 -> 27 us;
  // N = 8192, K = 28672, 896 blocks: 75 -> 58 us; with full rounds it keeps the shape: N = 8192, K = 16384, 512 blocks: 39
  // against 43 us here)
  if (M > 32 && M <= 64 && !((p.splits == 1 && tiles * 2 > cus && p.kb_per_split >= 8) || (p.splits == 2 && p.kb_per_split >= 16)) &&
      !(entries == 1 && p.kb_per_split >= 16 && mid_m_partial_round(plan_mid_m(M, N, K), cus)))
    return p;
  // (two ranges of eight: N = 16384, K = 2048: 14 -> 17 us; of sixteen: N = 14336, K = 4096: 29 -> 22 us; N = 12288, K = 4096: 28 -> 20 us)
  // 17..32 rows of a lone matrix: the decode kernels, except unsplit against very wide weights (M = 32: N = 24576,
  // K = 1536: 18.3 -> 15.1 us; N = 28672, K = 4096: 34.9 -> 30.9 us; N = 32768, K = 1024: 15.8 -> 12.7 us), and up to 24
  // rows only while K is short (M = 24, N = 28672, K = 4096: 34.0 -> 36.3 us, so not there; N = 20480, K = 3072: 24.8 -> 23.3 us)
  // (one range because the tiles fill the compute units, not because K is too short to split: N = 8192, K = 1024, 64 tiles,
  // 10.5 us here whatever M; M = 17 ... 32: 5.2-5.7 us on the decode kernels, 33 ... 64: 7.5-7.9 us on the staged-activation
  // kernel; N = 16384, K = 1024, 128 tiles, M = 48 / 64: 10.9 / 11.0 -> 8.1 / 8.5 us)
  if (M <= 32 && !(p.splits == 1 && tiles * 2 > cus && p.kb_per_split >= 8 && (M > 24 || KB <= 24))) return p;
  p.workspace_bytes = p.splits > 1 ? FG_WORKSPACE_COUNTER_BYTES + (size_t)tiles * p.splits * kSplitTile * kSplitTile * sizeof(float) : 0;
  p.use = true;
  return p;
}

template <int MODE>
int launch_pipe(GemmArgs a, const PipePlan& plan, void* workspace, hipStream_t stream) {
  using Cfg = TileCfg<kSplitTile, kSplitTile, kSplitWM, 2, kPipeStages>;
  a.tiles_m = (int)ceil_div(a.M, kSplitTile);
  a.tiles_n = (int)ceil_div(a.N, kSplitTile);
  a.splits = plan.splits;
  a.kb_per_split = plan.kb_per_split;
  a.split_counters = reinterpret_cast<unsigned int*>(workspace);
  a.split_partials = workspace && plan.splits > 1 ? reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(workspace) + FG_WORKSPACE_COUNTER_BYTES) : nullptr;
  a.split_partials_per_entry = (int64_t)a.tiles_m * a.tiles_n * a.splits * kSplitTile * kSplitTile;
  auto kern = fp8_gemm_kernel<kSplitTile, kSplitTile, kSplitWM, 2, MODE, true, true, kPipeStages>;
  static PerDeviceFlags lds_limit_raised = {};
  {
    const hipError_t e = raise_dynamic_lds_limit(lds_limit_raised, Cfg::kLdsBytes, reinterpret_cast<const void*>(kern));
    if (e != hipSuccess) FG_FAIL(FG_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", Cfg::kLdsBytes, hipGetErrorString(e));
  }
  const int64_t blocks = (int64_t)a.tiles_m * a.tiles_n * a.splits;
  FG_LAUNCH(kern, dim3((uint32_t)blocks, (uint32_t)(a.batch > 1 ? a.batch : 1)), dim3(Cfg::kThreads), Cfg::kLdsBytes, stream, a);
  FG_CHECK_LAUNCH("fp8_gemm_kernel (four stages)");
  return FG_OK;
}

// Parts of up to 16 rows in which the decode kernels take 17..512 rows of a lone problem (measurements at the call): two, four,
// eight ... parts of `rows` rows each (three, five and six were measured and are 20-60 % slower than the next power of
// two); the last part starts `back` rows early so that it ends with the last row, and the rows it shares with the part
// before are computed alike by both.
struct DecodeParts {
  int64_t parts, rows, back;  // parts == 0: not taken
};
DecodeParts decode_parts(int64_t M, int64_t N, int64_t K) {
  DecodeParts d = {0, 0, 0};
  const int64_t bytes = N * K;
  if (M > 16 && M <= 32 && N <= 6144) d.parts = 2;
  else if (M > 32 && M <= 64 && N <= 8192 && (bytes <= ((int64_t)13 << 20) || (N <= 3072 && bytes <= ((int64_t)26 << 20)))) d.parts = 4;
  else if (M > 64 && M <= 128 && N <= 4096 && bytes <= ((int64_t)23 << 19)) d.parts = 8;
  // (sixteen and thirty-two parts against the very smallest weights; us at M = 129 / 192 / 256, four 64-row parts on the
  // staged-activation kernel -> sixteen parts: N = 512, K = 7168: 11.1 / 11.7 / 11.8 -> 7.8 / 8.0 / 8.6; N = 256, K = 8192: 10.8 / 11.3 / 11.9 ->
  // 5.9 / 6.2 / 8.2; N = K = 1024: 7.1 / 7.4 / 7.5 -> 5.0 / 5.0 / 5.1; not N = 1024, K = 4096: 9.5 -> 10.0; M = 257 / 512 in thirty-two:
  // N = 256, K = 8192: 11.9 / 12.3 -> 8.2 / 9.8; N = K = 1024: 7.5 / 7.6 -> 5.9 / 6.6)
  else if (M > 128 && M <= 256 && (bytes <= ((int64_t)2 << 20) || (N <= 768 && bytes <= ((int64_t)6 << 20)))) d.parts = 16;
  else if (M > 256 && M <= 512 && N <= 4096 && bytes <= ((int64_t)2 << 20)) d.parts = 32;
  else return d;
  d.rows = ceil_div(M, d.parts);           // <= 16: M <= 16 * parts
  d.back = d.parts * d.rows - M;           // < parts: rows that the last part shares with the one before
  return d;
}

// Into how many equal parts of at most 64 rows the staged-activation kernel takes the rows of a lone problem above 64 rows
// (measurements at the call); 0: not at all.
int64_t row_parts(int64_t M, int64_t N, int64_t K) {
  const int64_t bytes = N * K;
  if (M > 64 && M <= 128 &&
      ((N <= 32768 && bytes <= ((int64_t)8 << 20)) || (N <= 3072 && bytes <= ((int64_t)34 << 20)) || (N <= 4096 && bytes <= ((int64_t)17 << 20))))
    return 2;
  // more parts only for the smallest weights, which every part reads again: us at M = 129 / 192 / 256, N = 512, K = 7168:
  // 16.7 / 17.5 / 18.2 -> 11.1 / 11.7 / 11.9; N = 1024, K = 4096: 14.8 / 15.2 / 15.8 -> 9.6 / 10.0 / 10.2; N = K = 2048: 12.6 / 12.7 / 13.0 ->
  // 9.0 / 9.6 / 9.7; up to 192 rows, N = 1280, K = 8192: 18.6 / 18.8 -> 14.9 / 16.3; N = 1024, K = 8192: 18.1 / 18.6 -> 16.0 / 17.2 (N = 2112,
  // K = 7168: 19.2 -> 20.9; N = K = 4096: 16.6 -> 23.2)
  // (very wide weights with one or two K-blocks lose: N = 65536, K = 128, M = 128: 11.9 -> 13.2; N = 32768, K = 128, M = 256: 9.8 -> 12.7;
  // N = 16384, K = 512, M = 129: 9.0 -> 10.8; N = 16384, K = 128, M = 257: 8.4 -> 10.8)
  if (M > 128 && M <= 256 && N <= 16384 && bytes <= ((int64_t)4 << 20)) return ceil_div(M, (int64_t)64);
  if (M > 128 && M <= 192 && N <= 8192 && bytes <= ((int64_t)10 << 20)) return 3;
  // (257..512 rows: N = 1024, K = 2048: 12.6 -> 9.4; N = 256, K = 8192: 17.2 / 18.4 -> 12.0 / 12.3 at 257 / 512 rows; N = 512, K = 7168:
  // 17.6 / 18.4 -> 15.2 / 17.0; N = 1024, K = 8192: 20.6 -> 21.2)
  if (M > 256 && M <= 512 && N <= 8192 && bytes <= ((int64_t)2 << 20)) return ceil_div(M, (int64_t)64);
  return 0;
}

// Whether the 33..64-row kernel is the one to take for the shape (it is compared with the K-split tile kernel and
// the decode kernels, which take the same shapes).
bool mid_m_preferred(const MidMPlan& mid, int64_t M, int64_t N, int64_t K) {
  (void)M;
  // 33..64 rows: always (measured against both alternatives on every DeepSeek-V3 and Llama-3 shape).  65..128 rows:
  // the splits' partial sums cost as much as the weights, which pays only while the weights are small: M = 128,
  // N = 6144, K = 4096: 31 -> 20 us; N = 7168, K = 2304: 19 -> 16 us; but N = 24576, K = 1536: 23 -> 28 us.
  return mid.use && (mid.tmx <= 4 || N * K <= (int64_t)28 << 20);
}

template <int MODE>
int launch_gemm(const GemmArgs& a, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  // K == 0 (an empty sum: zeros, or the bias) goes to the guarded tile kernel, whose K loop may be empty; the
  // kernels below all assume at least one K-block
  const bool direct = (a.K > 0) && (a.K % 128 == 0) && (a.ldx % 16 == 0) && (a.ldw % 16 == 0) &&
                      (a.ldx < (1 << 23)) && (a.ldw < (1 << 23)) &&
                      ((uintptr_t)a.X % 16 == 0) && ((uintptr_t)a.W % 16 == 0);
  // 17..128 rows against narrow or small weights: parts of up to 16 rows on the decode kernels in one launch (the entries of a
  // batch that shares the weights).  With 17 rows or more a decode block fetches 32 activation rows per 16-32 weight rows
  // through registers; with up to 16 the activations of its K range lie in LDS.  Every part reads the weights again, so
  // the more parts, the smaller the weights that stand it.
  // 17..32 rows in two parts, weights of up to 6144 rows; us at M = 17 / 24 / 32, before (decode kernels for 32 rows, or 32 rows
  // staged in the kernel of 33..64 rows) -> after: N = 2112, K = 7168: 10.2 / 10.8 / 10.8 -> 7.4 / 7.7 / 9.2; N = 3072, K = 8192: 11.8 / 12.4 / 12.7 ->
  // 8.6 / 10.1 / 10.3; N = 1024, K = 8192: 8.4 / 9.6 / 10.2 -> 6.2 / 6.5 / 9.2; N = 4096, K = 14336: 18.8 / 19.6 / 20.0 -> 17.4 / 17.4 / 17.4; N = 576,
  // K = 7168: 8.1 / 9.1 / 9.5 -> 5.7 / 6.0 / 6.3; N = K = 6144: 12.9 / 14.3 / 15.9 -> 11.7 / 12.1 / 13.4; N = 6144, K = 256: 4.3 -> 3.6.  Wider weights
  // lose (N = 7168, K = 2304: 7.1 -> 8.0; N = 10240, K = 8192: 23 -> 31; N = 28672, K = 4096: 27 -> 45).
  // 33..64 rows in four parts, up to 13 MB (26 MB with N <= 3072); M = 33 / 48 / 64, staged-activation kernel -> four parts:
  // N = 2112, K = 7168: 12.2 / 12.2 / 13.1 -> 10.7 / 10.8 / 13.1; N = 1536, K = 7168: 11.4 / 11.4 / 12.0 -> 7.9 / 7.6 / 8.8; N = 1280, K = 8192:
  // 11.7 / 11.7 / 12.2 -> 8.0 / 9.1 / 9.3; N = 1536, K = 12288: 16.5 / 16.8 / 17.9 -> 12.4 / 12.3 / 12.6; N = 8192, K = 1536: 11.4 / 11.4 / 15.0 ->
  // 8.0 / 8.2 / 8.7; N = 512, K = 7168: 10.2 / 10.2 / 10.8 -> 5.8 / 5.8 / 6.1; not N = K = 4096: 10.0 -> 10.7, N = 6144, K = 4096: 13.1 -> 14.5,
  // N = 32768, K = 256: 5.8 -> 8.6.
  // 65..128 rows in eight parts, up to 11.5 MB and 4096 rows; M = 65 / 96 / 128, two halves on the staged-activation kernel ->
  // eight parts: N = 512, K = 7168: 11.0 / 11.2 / 11.7 -> 5.8 / 6.2 / 6.3; N = K = 2048: 8.8 / 8.8 / 9.4 -> 6.6 / 6.7 / 6.8; N = 1024, K = 8192:
  // 11.6 / 11.7 / 12.3 -> 8.8 / 9.9 / 10.0; N = 1536, K = 7168: 14.1 / 14.4 / 15.7 -> 10.9 / 11.1 / 13.7; not N = 2112, K = 7168: 15.7 -> 19.7.
  if (const DecodeParts dp = direct && a.batch <= 1 ? decode_parts(a.M, a.N, a.K) : DecodeParts{0, 0, 0}; dp.parts > 1) {
    const int64_t parts = dp.parts, stride = dp.rows, rows = dp.rows;
    const SmallMPlan sp = plan_small_m(rows, a.N, a.K, parts);
    const size_t per_entry = sp.splits > 1 ? sp.workspace_bytes - FG_WORKSPACE_COUNTER_BYTES : 0;
    const bool fits = sp.use && (sp.splits == 1 || (workspace != nullptr && (uintptr_t)workspace % 16 == 0 &&
                                                    workspace_bytes >= FG_WORKSPACE_COUNTER_BYTES + (size_t)parts * per_entry &&
                                                    (size_t)parts * sp.n_chunks * sizeof(unsigned int) <= FG_WORKSPACE_COUNTER_BYTES));
    if (fits) {
      GemmArgs h = a;
      const int64_t c_elem = a.c_dtype == FG_F32 ? 4 : (a.c_dtype == FG_BF16 || a.c_dtype == FG_F16) ? 2 : 1;
      h.M = (int)rows;
      h.batch = (int)parts;
      h.x_batch_bytes = stride * a.ldx;
      h.w_batch_bytes = 0;
      h.c_batch_bytes = stride * a.ldc * c_elem;
      h.xs_batch_stride = MODE == kModeBlock ? stride * a.xs_rs : (a.xs_per_row ? stride : 0);
      h.ws_batch_stride = 0;
      h.last_x_back_bytes = dp.back * a.ldx;
      h.last_c_back_bytes = dp.back * a.ldc * c_elem;
      h.last_xs_back = MODE == kModeBlock ? dp.back * a.xs_rs : (a.xs_per_row ? dp.back : 0);
      return launch_small_m(h, MODE, sp, workspace, workspace_bytes, stream);
    }
  }
  // 65..128 rows against small weights: the staged-activation kernel over the two halves of the rows in one launch (the
  // halves are the entries of a batch that shares the weights; 33..48 rows stage 48, 49..64 stage 64).  The weights are
  // read twice, which small ones stand: us at M = 65 / 96 / 128, K-split tile kernel -> here: N = 2112, K = 7168:
  // 19.3 / 19.6 / 19.9 -> 15.8 / 16.2 / 17.3; N = K = 4096: 15.9 / 16.2 / 16.7 -> 14.7 / 13.9 / 15.0; N = 1024, K = 8192: 17.9 / 18.4 / 19.0 ->
  // 11.7 / 11.8 / 12.4; N = 8192, K = 1024: 10.7 / 11.0 / 11.2 -> 7.7 / 8.0 / 8.3; N = 2048, K = 16384: 23.3 / 25.1 / 26.2 -> 20.9 / 21.3 / 23.3.
  // Wider or larger weights lose (N = 4608, K = 7168: 20 -> 33; N = 7168, K = 2304: 13.8 -> 14.4; N = 5120, K = 5120: 17.8 -> 20.2;
  // N = 2304, K = 16384: 24.0 -> 26.5).
  if (const int64_t parts = direct && a.batch <= 1 ? row_parts(a.M, a.N, a.K) : 0; parts > 1) {
    const int64_t rows = ceil_div((int64_t)a.M, parts);
    const MidMPlan mh = plan_mid_m(rows, a.N, a.K, parts);
    const size_t per_entry = mh.splits > 1 ? mh.workspace_bytes - FG_WORKSPACE_COUNTER_BYTES : 0;
    const bool fits = mh.use && (mh.splits == 1 || (workspace != nullptr && (uintptr_t)workspace % 16 == 0 &&
                                                    workspace_bytes >= FG_WORKSPACE_COUNTER_BYTES + (size_t)parts * per_entry &&
                                                    (size_t)parts * mh.n_chunks * sizeof(unsigned int) <= FG_WORKSPACE_COUNTER_BYTES));
    if (fits) {
      GemmArgs h = a;
      const int64_t c_elem = a.c_dtype == FG_F32 ? 4 : (a.c_dtype == FG_BF16 || a.c_dtype == FG_F16) ? 2 : 1;
      h.M = (int)rows;
      h.batch = (int)parts;
      h.last_entry_rows = (int)(a.M - (parts - 1) * rows);
      h.x_batch_bytes = rows * a.ldx;
      h.w_batch_bytes = 0;
      h.c_batch_bytes = rows * a.ldc * c_elem;
      h.xs_batch_stride = MODE == kModeBlock ? rows * a.xs_rs : (a.xs_per_row ? rows : 0);
      h.ws_batch_stride = 0;
      return launch_mid_m(h, MODE, mh, workspace, workspace_bytes, stream);
    }
  }
  if (direct) {
    const MidMPlan mid = plan_mid_m(a.M, a.N, a.K);
    // (65..128 rows: the 128-row variant of that kernel loses to the four-stage tile kernel below on every shape
    // measured -- M = 128: N = 2112, K = 7168: 24.0 against 19.9 us; 7168 x 2304: 16.4 against 14.6; 4096 x 4096: 18.4
    // against 16.8 -- and only serves batches now)
    const bool mid_takes = mid.use && mid.tmx <= 4;
    if (a.M > 16 && a.M <= 48) {
      // very wide weights against short K: a wavefront per 16 weight rows with the block's activations in LDS
      // (N = 24576, K = 1536, M = 17 / 24 / 32 / 40: 15.1 / 13.8 / 13.7 / 14.2 us on the kernels below)
      const SmallMPlan sp = plan_small_m(a.M, a.N, a.K);
      if (sp.use && sp.own) return launch_small_m(a, MODE, sp, workspace, workspace_bytes, stream);
    }
    if (a.M <= 64) {  // the four-stage tile kernel where its planner prefers it to the staged-activation and decode kernels
      const PipePlan pp = plan_pipe(a.M, a.N, a.K, MODE == kModeBlock ? a.xs_rs : 0);
      const bool ws_ok = pp.splits == 1 || (workspace != nullptr && workspace_bytes >= pp.workspace_bytes && (uintptr_t)workspace % 16 == 0);
      if (pp.use && ws_ok) return launch_pipe<MODE>(a, pp, workspace, stream);
    }
    if (mid_takes && (mid.splits == 1 || (workspace != nullptr && workspace_bytes >= mid.workspace_bytes &&
                                          (uintptr_t)workspace % 16 == 0)))
      return launch_mid_m(a, MODE, mid, workspace, workspace_bytes, stream);
    {
      const PipePlan pp = plan_pipe(a.M, a.N, a.K, MODE == kModeBlock ? a.xs_rs : 0);
      const bool ws_ok = pp.splits == 1 || (workspace != nullptr && workspace_bytes >= pp.workspace_bytes && (uintptr_t)workspace % 16 == 0);
      if (pp.use && ws_ok && !mid_takes) return launch_pipe<MODE>(a, pp, workspace, stream);
    }
    const TileSplitPlan ts = plan_tile_split(a.M, a.N, a.K);
    if (ts.use && workspace != nullptr && workspace_bytes >= ts.workspace_bytes && (uintptr_t)workspace % 16 == 0)
      return launch_tile_split<MODE>(a, ts, workspace, stream);
    const SmallMPlan plan = plan_small_m(a.M, a.N, a.K);
    if (plan.use) return launch_small_m(a, MODE, plan, workspace, workspace_bytes, stream);
  }
  {
    const int64_t tiles128 = ceil_div(a.M, 128) * ceil_div(a.N, 128);
    // 257..512 tiles of 128 x 128 with K up to 4096: at most the 512 workgroups that are
    // resident at a time, two on each compute unit (560 tiles: M = 1280, N = 7168, K = 2304 went from 36 to 51 us); the persistent kernel has a quarter of the tiles and spends its
    // time filling and draining.  Measured: M = 256, N = 24576, K = 1536: 27.7 -> 23.4 us; M = 768, N = 7168, K = 2304:
    // 34.8 -> 28.9; N = 6144, K = 4096: 50.0 -> 43.4; M = 1024, N = 7168, K = 2304: 35.3 -> 29.6.
    // The tile count decides, whatever M: M = 2048, N = 3072, K = 2048: 34.0 -> 24.8 us; M = 3072, N = K = 2048: 34.0 -> 24.2;
    // M = 2048, N = K = 4096: 51.0 -> 45.2.
    // With longer K the persistent kernel, which shares tiles between compute units through the workspace, is ahead: the rule
    // once reached to K = 8192 for up to 448 tiles, and without that M = 256, N = 20480, K = 8192 goes from 100 to 72 us; M = 512,
    // N = 10240: 92 -> 65; M = 384, N = 14336: 91 -> 78; M = 768, N = 7168: 85 -> 65; M = 512, N = 9216, K = 6144: 73 -> 55; M = 256,
    // N = 20480, K = 5120: 70 -> 56; M = 1024, N = 4608, K = 7168: 74 -> 58; M = 2048, N = 2112, K = 7168: 70 -> 62 (of 105 cases
    // measured, five lose, by 3-8 %: M = 768, N = 20480, K = 5120: 73 -> 78).
    if (direct && a.M > 128 && tiles128 > 256 && tiles128 <= 512 && a.KB <= 32)
      return launch_cfg<128, 128, 4, 2, MODE, true>(a, stream);  // eight wavefronts: 7-13 % faster than four on these shapes
  }
  const bool big = a.M > 128;
  if (direct && pingpong_takes(a, MODE, workspace, workspace_bytes)) return launch_pingpong(a, MODE, workspace, workspace_bytes, stream);
  if (big) {
    // Row/column modes that the persistent kernel does not take (fp32 or fp8 results, rows that take no 16-byte
    // stores, K not a multiple of 128): 128 x 128 tiles.  The 256 x 256 instantiation of these modes does not fit the
    // registers (40 spilled): fp32 results, M = 4096, N = 7168: K = 2304 438 -> 124 us, K = 16384 3129 -> 467 us;
    // K = 4160 (loads through registers), M = N = 4096, bf16: fp8 382 -> 107 us, int8 755 -> 129 us.
    if (MODE != kModeBlock)
      return direct ? launch_cfg<128, 128, 4, 2, MODE, true>(a, stream) : launch_cfg<128, 128, 4, 2, MODE, false>(a, stream);
    // block scales through registers: 256 x 256 tiles once they fill the compute units (M = N = 4096, K = 4160: 98
    // against 120 us), 128 x 128 below (M = 1024: 88 -> 43 us; M = 256: 83 -> 34 us)
    if (!direct && ceil_div(a.M, 256) * ceil_div(a.N, 256) < cu_count()) return launch_cfg<128, 128, 4, 2, MODE, false>(a, stream);
    return direct ? launch_cfg<256, 256, 4, 2, MODE, true>(a, stream)
                  : launch_cfg<256, 256, 4, 2, MODE, false>(a, stream);
  }
  return direct ? launch_cfg<128, 128, 2, 2, MODE, true>(a, stream)
                : launch_cfg<128, 128, 2, 2, MODE, false>(a, stream);
}

int check_common(const void* A, const void* B, const void* C, int64_t lda, int64_t ldb, int64_t ldc,
                 int64_t M, int64_t N, int64_t K, const char* who) {
  if (M < 0 || N < 0 || K < 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: negative size", who);
  if (M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFF00) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: size exceeds 2^31", who);
  if (M == 0 || N == 0) return 1;
  if (!C) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null output", who);
  if (K > 0 && (!A || !B)) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null operand", who);
  if (lda < K || ldb < K || ldc < N) FG_FAIL(FG_ERR_INVALID_ARG, "%s: leading dimension smaller than row length", who);
  return 0;
}

}  // namespace
}  // namespace fg

extern "C" size_t fg_block_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  // the largest any kernel that may take the shape can use
  size_t need = fg::plan_tile_split(M, N, K).workspace_bytes;
  const fg::PipePlan pipe = fg::plan_pipe(M, N, K, 0);
  if (pipe.use && pipe.workspace_bytes > need) need = pipe.workspace_bytes;
  const fg::SmallMPlan plan = fg::plan_small_m(M, N, K);
  if (plan.use && plan.workspace_bytes > need) need = plan.workspace_bytes;
  const fg::MidMPlan mid = fg::plan_mid_m(M, N, K);
  if (mid.use && mid.workspace_bytes > need) need = mid.workspace_bytes;
  if (const fg::DecodeParts dp = fg::decode_parts(M, N, K); dp.parts > 1) {  // the decode kernels over parts of the rows
    const fg::SmallMPlan sp = fg::plan_small_m(dp.rows, N, K, dp.parts);
    if (sp.use && sp.splits > 1) {
      const size_t all = FG_WORKSPACE_COUNTER_BYTES + (size_t)dp.parts * (sp.workspace_bytes - FG_WORKSPACE_COUNTER_BYTES);
      if (all > need) need = all;
    }
  }
  if (const int64_t parts = fg::row_parts(M, N, K); parts > 1) {  // the same kernel over equal parts of the rows
    const fg::MidMPlan mh = fg::plan_mid_m(fg::ceil_div(M, parts), N, K, parts);
    if (mh.use && mh.splits > 1) {
      const size_t both = FG_WORKSPACE_COUNTER_BYTES + (size_t)parts * (mh.workspace_bytes - FG_WORKSPACE_COUNTER_BYTES);
      if (both > need) need = both;
    }
  }
  const size_t pp = fg::pingpong_workspace_bytes(M, N, K);
  return pp > need ? pp : need;
}
extern "C" size_t fg_scaled_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  return fg_block_fp8_gemm_workspace_bytes(M, N, K);
}

namespace fg {
namespace {
int block_fp8_gemm(const char* who, int scales_pow2, const void* A, int64_t lda, const void* B, int64_t ldb,
                                 const float* As, int64_t as_row_stride, int64_t as_col_stride,
                                 const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride,
                                 void* C, int64_t ldc, int c_dtype,
                                 int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  if (block_n < 1 || block_k < 1)
    FG_FAIL(FG_ERR_INVALID_ARG, "%s: scale block %lld x %lld", who, (long long)block_n, (long long)block_k);
  if (c_dtype != FG_BF16 && c_dtype != FG_F16 && c_dtype != FG_F32)
    FG_FAIL(FG_ERR_INVALID_ARG, "%s: c_dtype %d", who, c_dtype);
  int rc = check_common(A, B, C, lda, ldb, ldc, M, N, K, who);
  if (rc < 0) return rc;
  if (rc == 1) return FG_OK;
  if (K > 0 && (!As || !Bs)) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null scale pointer", who);
  GemmArgs a = {};
  a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.C = C;
  a.xs = As; a.ws = Bs; a.bias = nullptr;
  a.ldx = lda; a.ldw = ldb; a.ldc = ldc;
  a.xs_rs = as_row_stride; a.xs_cs = as_col_stride; a.ws_rs = bs_row_stride; a.ws_cs = bs_col_stride;
  a.M = (int)M; a.N = (int)N; a.K = (int)K; a.KB = (int)ceil_div(K, 128);
  a.c_dtype = c_dtype;
  a.scales_pow2 = scales_pow2;
  // the matrix-instruction kernels apply one scale product per 128 x 128 block; every other block size takes the
  // plain kernel (the host side restates multiples of 128 at 128 x 128 first, so they do not come here)
  if (block_n != 128 || block_k != 128) return launch_anyblock(a, block_n, block_k, (hipStream_t)stream);
  return launch_gemm<kModeBlock>(a, workspace, workspace_bytes, (hipStream_t)stream);
}
}  // namespace
}  // namespace fg

extern "C" int fg_block_fp8_gemm(const void* A, int64_t lda, const void* B, int64_t ldb,
                                 const float* As, int64_t as_row_stride, int64_t as_col_stride,
                                 const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride,
                                 void* C, int64_t ldc, int c_dtype,
                                 int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  return fg::block_fp8_gemm("fg_block_fp8_gemm", 0, A, lda, B, ldb, As, as_row_stride, as_col_stride, Bs, bs_row_stride, bs_col_stride,
                            C, ldc, c_dtype, M, N, K, block_n, block_k, workspace, workspace_bytes, stream);
}

extern "C" int fg_block_fp8_gemm_pow2_scales(const void* A, int64_t lda, const void* B, int64_t ldb,
                                             const float* As, int64_t as_row_stride, int64_t as_col_stride,
                                             const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride,
                                             void* C, int64_t ldc, int c_dtype,
                                             int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k,
                                             void* workspace, size_t workspace_bytes, void* stream) {
  return fg::block_fp8_gemm("fg_block_fp8_gemm_pow2_scales", 1, A, lda, B, ldb, As, as_row_stride, as_col_stride, Bs, bs_row_stride,
                            bs_col_stride, C, ldc, c_dtype, M, N, K, block_n, block_k, workspace, workspace_bytes, stream);
}

// ---------------------------------------------------------------------------------------------
// fg_block_fp8_gemm for callers that cannot allocate: the workspace is a device array built into the library.
// ---------------------------------------------------------------------------------------------
namespace fg {
namespace {

constexpr size_t kScratchBytes = FG_NOALLOC_SCRATCH_BYTES;
// Counters (first FG_WORKSPACE_COUNTER_BYTES), split-K partial sums and transposed activation scales of the
// launches made through fg_block_fp8_gemm_noalloc.  One copy per GPU, at an address of its own on each; in host
// code the name is only a handle for hipGetSymbolAddress.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// device address of `scratch` on each device, looked up on the first call made with that device current
struct ScratchTable {
  std::mutex lock;
  void* ptr[kMaxDevices] = {};
};
ScratchTable& scratch_table() {
  static ScratchTable t;
  return t;
}

// Address of the current device's copy (looked up once per device).  Nothing is enqueued here: a file-scope device
// array without an initialiser is zero when the code object is loaded, which is the state the counter area has to
// start from, and every launch leaves the counters zero again.  (A fill kernel on the first caller's stream would be
// ordered against that stream only, and recorded into the caller's graph if the first call were made under capture.)
int scratch_of_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) FG_FAIL(FG_ERR_LAUNCH, "fg_block_fp8_gemm_noalloc: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) FG_FAIL(FG_ERR_UNSUPPORTED, "fg_block_fp8_gemm_noalloc: device index %d (at most %d devices)", dev, kMaxDevices);
  ScratchTable& t = scratch_table();
  std::lock_guard<std::mutex> guard(t.lock);
  if (t.ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      FG_FAIL(FG_ERR_LAUNCH, "fg_block_fp8_gemm_noalloc: hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    t.ptr[dev] = p;
  }
  *out = t.ptr[dev];
  return FG_OK;
}

}  // namespace
}  // namespace fg

extern "C" int fg_block_fp8_gemm_noalloc(const void* A, int64_t lda, const void* B, int64_t ldb,
                                         const float* As, int64_t as_row_stride, int64_t as_col_stride,
                                         const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride,
                                         void* C, int64_t ldc, int c_dtype,
                                         int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k, void* stream) {
  using namespace fg;
  if (M < 0 || N < 0 || K < 0) FG_FAIL(FG_ERR_INVALID_ARG, "fg_block_fp8_gemm_noalloc: negative size");
  const size_t need = fg_block_fp8_gemm_workspace_bytes(M, N, K);
  if (need > kScratchBytes)
    FG_FAIL(FG_ERR_WORKSPACE,
            "fg_block_fp8_gemm_noalloc: M = %lld, N = %lld, K = %lld wants %zu bytes of workspace and the built-in buffer has "
            "%zu; call fg_block_fp8_gemm with a workspace of the caller's",
            (long long)M, (long long)N, (long long)K, need, kScratchBytes);
  void* ws = nullptr;
  const int rc = scratch_of_current_device(&ws);
  if (rc != FG_OK) return rc;
  return fg_block_fp8_gemm(A, lda, B, ldb, As, as_row_stride, as_col_stride, Bs, bs_row_stride, bs_col_stride, C, ldc, c_dtype,
                           M, N, K, block_n, block_k, ws, kScratchBytes, stream);
}

extern "C" size_t fg_batched_block_fp8_gemm_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K) {
  size_t need = fg_block_fp8_gemm_workspace_bytes(M, N, K);
  if (batch > 1 && M >= 1 && M <= 32) {
    const fg::SmallMPlan plan = fg::plan_small_m(M, N, K, batch);
    if (plan.use && plan.splits > 1) {
      const size_t all = FG_WORKSPACE_COUNTER_BYTES + (size_t)batch * (plan.workspace_bytes - FG_WORKSPACE_COUNTER_BYTES);
      if (all > need) need = all;
    }
  }
  if (batch > 1 && M > 32 && M <= 128) {
    const fg::MidMPlan mid = fg::plan_mid_m(M, N, K, batch);
    if (mid.use && mid.splits > 1) {
      const size_t all = FG_WORKSPACE_COUNTER_BYTES + (size_t)batch * (mid.workspace_bytes - FG_WORKSPACE_COUNTER_BYTES);
      if (all > need) need = all;
    }
  }
  if (batch > 1) {
    const fg::PipePlan pipe = fg::plan_pipe(M, N, K, 0, batch);
    if (pipe.use && pipe.workspace_bytes > need) need = pipe.workspace_bytes;
  }
  return need;
}

extern "C" int fg_batched_block_fp8_gemm(const void* A, int64_t lda, int64_t a_batch_stride,
                                         const void* B, int64_t ldb, int64_t b_batch_stride,
                                         const float* As, int64_t as_row_stride, int64_t as_col_stride, int64_t as_batch_stride,
                                         const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride, int64_t bs_batch_stride,
                                         void* C, int64_t ldc, int64_t c_batch_stride, int c_dtype,
                                         int64_t batch, int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k,
                                         void* workspace, size_t workspace_bytes, void* stream) {
  using namespace fg;
  if (batch < 0) FG_FAIL(FG_ERR_INVALID_ARG, "fg_batched_block_fp8_gemm: negative batch count");
  if (a_batch_stride < 0 || b_batch_stride < 0 || as_batch_stride < 0 || bs_batch_stride < 0 || c_batch_stride < 0)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_batched_block_fp8_gemm: negative batch stride");
  const size_t c_elem = c_dtype == FG_F32 ? 4 : 2;
  // Entries that would each leave most of the GPU idle (fewer than 192 tiles of 256 x 256) go out together: one
  // launch of the tile kernel, blockIdx.y = entry.  Measured on [b, h, r] x [h, d, r], one launch per head -> one
  // launch: h = 8, r = 4096, d = 1024: b = 128: 140 -> 41 us, b = 4096: 403 -> 200 us (1.37 PFLOP/s);
  // h = 16, r = 7168: b = 128: 354 -> 68 us, b = 4096: 926 -> 787 us.
  {
    const bool direct = K > 0 && K % 128 == 0 && lda % 16 == 0 && ldb % 16 == 0 && lda < (1 << 23) && ldb < (1 << 23) &&
                        (uintptr_t)A % 16 == 0 && (uintptr_t)B % 16 == 0 && a_batch_stride % 16 == 0 && b_batch_stride % 16 == 0;
    const int64_t big_tiles = ceil_div(M, 256) * ceil_div(N, 256);
    if (batch > 1 && batch <= 65535 && direct && big_tiles < 192 && block_n == 128 && block_k == 128 &&
        (c_dtype == FG_BF16 || c_dtype == FG_F16 || c_dtype == FG_F32) && As && Bs) {
      int rc = check_common(A, B, C, lda, ldb, ldc, M, N, K, "fg_batched_block_fp8_gemm");
      if (rc < 0) return rc;
      if (rc == 1) return FG_OK;
      GemmArgs a = {};
      a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.C = C;
      a.xs = As; a.ws = Bs; a.bias = nullptr;
      a.ldx = lda; a.ldw = ldb; a.ldc = ldc;
      a.xs_rs = as_row_stride; a.xs_cs = as_col_stride; a.ws_rs = bs_row_stride; a.ws_cs = bs_col_stride;
      a.M = (int)M; a.N = (int)N; a.K = (int)K; a.KB = (int)(K / 128);
      a.c_dtype = c_dtype;
      a.batch = (int)batch;
      a.x_batch_bytes = a_batch_stride; a.w_batch_bytes = b_batch_stride; a.c_batch_bytes = c_batch_stride * (int64_t)c_elem;
      a.xs_batch_stride = as_batch_stride; a.ws_batch_stride = bs_batch_stride;
      // up to 32 rows: the weight-streaming kernels with the entry in blockIdx.y, when the workspace holds every
      // entry's partial sums and the counter area every entry's counters; else (and above 32 rows) the tile kernel
      if (M <= 32) {
        const SmallMPlan plan = plan_small_m(M, N, K, batch);
        const size_t per_entry = plan.splits > 1 ? plan.workspace_bytes - FG_WORKSPACE_COUNTER_BYTES : 0;
        const bool fits = plan.splits == 1 ||
                          (workspace != nullptr && (uintptr_t)workspace % 16 == 0 &&
                           workspace_bytes >= FG_WORKSPACE_COUNTER_BYTES + (size_t)batch * per_entry &&
                           (size_t)batch * plan.n_chunks * sizeof(unsigned int) <= FG_WORKSPACE_COUNTER_BYTES);
        if (plan.use && fits) return launch_small_m(a, kModeBlock, plan, workspace, workspace_bytes, (hipStream_t)stream);
      }
      {
        // few tiles in the whole batch: the four-stage tile kernel, K split over blocks until the compute units are full
        const PipePlan pp = plan_pipe(M, N, K, as_row_stride, batch);
        const bool fits = pp.splits == 1 || (workspace != nullptr && (uintptr_t)workspace % 16 == 0 && workspace_bytes >= pp.workspace_bytes);
        if (pp.use && fits) return launch_pipe<kModeBlock>(a, pp, workspace, (hipStream_t)stream);
      }
      if (M > 32 && M <= 128) {  // the staged-activation kernel, entry in blockIdx.z, under the same conditions
        const MidMPlan mid = plan_mid_m(M, N, K, batch);
        const size_t per_entry = mid.splits > 1 ? mid.workspace_bytes - FG_WORKSPACE_COUNTER_BYTES : 0;
        const bool fits = mid.splits == 1 ||
                          (workspace != nullptr && (uintptr_t)workspace % 16 == 0 &&
                           workspace_bytes >= FG_WORKSPACE_COUNTER_BYTES + (size_t)batch * per_entry &&
                           (size_t)batch * mid.n_chunks * sizeof(unsigned int) <= FG_WORKSPACE_COUNTER_BYTES);
        // 65..128 rows: measured against the tile kernel on the same batch, b = 128: 8 x [1024, 4096]: 41 -> 26 us,
        // 16 x [1024, 7168]: 67 -> 81 us
        const bool small_enough = mid.tmx <= 4 || (int64_t)batch * N * K <= (int64_t)64 << 20;
        if (mid_m_preferred(mid, M, N, K) && small_enough && fits) return launch_mid_m(a, kModeBlock, mid, workspace, workspace_bytes, (hipStream_t)stream);
      }
      // 256 x 256 tiles once the batch has one for every compute unit (measured, h = 8, r = 4096, d = 1024, 128-row against
      // 256-row tiles: b = 1024: 54 against 74 us; b = 2048: 101 against 84; b = 4096: 208 against 160 us = 1.72 PFLOP/s)
      if (batch * big_tiles >= 256) return launch_cfg<256, 256, 4, 2, kModeBlock, true>(a, (hipStream_t)stream);
      return launch_cfg<128, 128, 2, 2, kModeBlock, true>(a, (hipStream_t)stream);
    }
  }
  // One launch per matrix, in batch order on the caller's stream: each is the plain GEMM of its operands (same
  // kernels, same bits), and launches that follow each other on a stream may share the workspace.
  for (int64_t i = 0; i < batch; ++i) {
    const int rc = fg_block_fp8_gemm(
        A ? (const uint8_t*)A + i * a_batch_stride : nullptr, lda, B ? (const uint8_t*)B + i * b_batch_stride : nullptr, ldb,
        As ? As + i * as_batch_stride : nullptr, as_row_stride, as_col_stride,
        Bs ? Bs + i * bs_batch_stride : nullptr, bs_row_stride, bs_col_stride,
        C ? (uint8_t*)C + (size_t)(i * c_batch_stride) * c_elem : nullptr, ldc, c_dtype, M, N, K, block_n, block_k,
        workspace, workspace_bytes, stream);
    if (rc != FG_OK) return rc;
  }
  return FG_OK;
}

extern "C" size_t fg_grouped_block_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  (void)N;
  return fg::grouped_workspace_bytes(M, K);
}

extern "C" int fg_grouped_block_fp8_gemm(const void* A, int64_t lda,
                                         const void* B, int64_t ldb, int64_t b_group_stride,
                                         const float* As, int64_t as_row_stride, int64_t as_col_stride,
                                         const float* Bs, int64_t bs_row_stride, int64_t bs_col_stride, int64_t bs_group_stride,
                                         const int32_t* group_ends, int64_t n_groups,
                                         const int32_t* row_index, int64_t index_div, int64_t a_rows,
                                         int64_t c_rows, const float* row_weight,
                                         void* C, int64_t ldc, int c_dtype,
                                         int64_t M, int64_t N, int64_t K, int64_t block_n, int64_t block_k,
                                         void* workspace, size_t workspace_bytes, void* stream) {
  using namespace fg;
  const char* const who = "fg_grouped_block_fp8_gemm";
  if (block_n != 128 || block_k != 128)
    FG_FAIL(FG_ERR_UNSUPPORTED, "%s: only 128x128 scale blocks are implemented (got %lld x %lld)", who,
            (long long)block_n, (long long)block_k);
  if (c_dtype != FG_BF16 && c_dtype != FG_F16) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: the result must be bf16 or fp16 (c_dtype %d)", who, c_dtype);
  if (n_groups <= 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: %lld groups", who, (long long)n_groups);
  int rc = check_common(A, B, C, lda, ldb, ldc, M, N, K, who);
  if (rc < 0) return rc;
  if (rc == 1) return FG_OK;
  if (!group_ends) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null group table", who);
  if (c_rows < 0 || c_rows > 0x7FFFFFFF || (c_rows > 0 && !row_index))
    FG_FAIL(FG_ERR_INVALID_ARG, "%s: c_rows = %lld (scattered results need row_index)", who, (long long)c_rows);
  if (row_weight && c_rows == 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: row_weight needs scattered results (c_rows > 0)", who);
  if (K == 0 || K % 128 != 0) FG_FAIL(FG_ERR_UNSUPPORTED, "%s: K = %lld is not a positive multiple of 128", who, (long long)K);
  if (!As || !Bs) FG_FAIL(FG_ERR_INVALID_ARG, "%s: null scale pointer", who);
  if (b_group_stride < 0 || bs_group_stride < 0) FG_FAIL(FG_ERR_INVALID_ARG, "%s: negative group stride", who);
  if (!(lda % 16 == 0 && ldb % 16 == 0 && lda < (1 << 23) && ldb < (1 << 23) && (uintptr_t)A % 16 == 0 &&
        (uintptr_t)B % 16 == 0 && b_group_stride % 16 == 0))
    FG_FAIL(FG_ERR_UNSUPPORTED, "%s: operands must be 16-byte aligned with row and group strides that are multiples of 16 below 2^23", who);
  GemmArgs a = {};
  a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.C = C;
  a.xs = As; a.ws = Bs; a.bias = nullptr;
  a.ldx = lda; a.ldw = ldb; a.ldc = ldc;
  a.xs_rs = as_row_stride; a.xs_cs = as_col_stride; a.ws_rs = bs_row_stride; a.ws_cs = bs_col_stride;
  a.M = (int)M; a.N = (int)N; a.K = (int)K; a.KB = (int)(K / 128);
  a.c_dtype = c_dtype;
  GroupedGemm grouped = {group_ends, n_groups, b_group_stride, bs_group_stride, row_index, index_div, (row_index && index_div != 0) ? a_rows : M,
                         c_rows, row_weight};
  return launch_grouped(a, grouped, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int fg_scaled_fp8_gemm(const void* A, int64_t lda, const void* B, int64_t ldb,
                                  const float* a_scale, int a_scale_per_row,
                                  const float* b_scale, int b_scale_per_col,
                                  const void* bias, int bias_dtype,
                                  void* C, int64_t ldc, int c_dtype,
                                  int64_t M, int64_t N, int64_t K,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  using namespace fg;
  if (c_dtype != FG_BF16 && c_dtype != FG_F16 && c_dtype != FG_F32 && c_dtype != FG_FP8_E4M3FN)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_scaled_fp8_gemm: c_dtype %d", c_dtype);
  if (bias && bias_dtype != FG_BF16 && bias_dtype != FG_F16 && bias_dtype != FG_F32)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_scaled_fp8_gemm: bias_dtype %d", bias_dtype);
  int rc = check_common(A, B, C, lda, ldb, ldc, M, N, K, "fg_scaled_fp8_gemm");
  if (rc < 0) return rc;
  if (rc == 1) return FG_OK;
  if (!a_scale || !b_scale) FG_FAIL(FG_ERR_INVALID_ARG, "fg_scaled_fp8_gemm: null scale pointer");
  GemmArgs a = {};
  a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.C = C;
  a.xs = a_scale; a.ws = b_scale; a.bias = bias;
  a.ldx = lda; a.ldw = ldb; a.ldc = ldc;
  a.M = (int)M; a.N = (int)N; a.K = (int)K; a.KB = (int)ceil_div(K, 128);
  a.c_dtype = c_dtype; a.bias_dtype = bias_dtype;
  a.xs_per_row = a_scale_per_row; a.ws_per_col = b_scale_per_col;
  return launch_gemm<kModeRowCol>(a, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" size_t fg_scaled_int8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  return fg_block_fp8_gemm_workspace_bytes(M, N, K);
}

extern "C" int fg_scaled_int8_gemm(const void* A, int64_t lda, const void* B, int64_t ldb,
                                   const float* a_scale, int a_scale_per_row,
                                   const float* b_scale, int b_scale_per_col,
                                   const void* bias, int bias_dtype,
                                   void* C, int64_t ldc, int c_dtype,
                                   int64_t M, int64_t N, int64_t K,
                                   void* workspace, size_t workspace_bytes, void* stream) {
  using namespace fg;
  if (c_dtype != FG_BF16 && c_dtype != FG_F16 && c_dtype != FG_F32)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_scaled_int8_gemm: c_dtype %d", c_dtype);
  if (bias && bias_dtype != FG_BF16 && bias_dtype != FG_F16 && bias_dtype != FG_F32)
    FG_FAIL(FG_ERR_INVALID_ARG, "fg_scaled_int8_gemm: bias_dtype %d", bias_dtype);
  int rc = check_common(A, B, C, lda, ldb, ldc, M, N, K, "fg_scaled_int8_gemm");
  if (rc < 0) return rc;
  if (rc == 1) return FG_OK;
  if (!a_scale || !b_scale) FG_FAIL(FG_ERR_INVALID_ARG, "fg_scaled_int8_gemm: null scale pointer");
  GemmArgs a = {};
  a.X = (const uint8_t*)A; a.W = (const uint8_t*)B; a.C = C;
  a.xs = a_scale; a.ws = b_scale; a.bias = bias;
  a.ldx = lda; a.ldw = ldb; a.ldc = ldc;
  a.M = (int)M; a.N = (int)N; a.K = (int)K; a.KB = (int)ceil_div(K, 128);
  a.c_dtype = c_dtype; a.bias_dtype = bias_dtype;
  a.xs_per_row = a_scale_per_row; a.ws_per_col = b_scale_per_col;
  // the dispatch of the fp8 operands with row and column scales: the kernels take the operand type as a mode, and
  // every exchange of partial sums adds int32 as int32
  return launch_gemm<kModeRowColI8>(a, workspace, workspace_bytes, (hipStream_t)stream);
}
