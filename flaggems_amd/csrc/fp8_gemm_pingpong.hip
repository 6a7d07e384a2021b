// Persistent "ping-pong" FP8 GEMM for gfx950: 256 x 256 output tiles, 8 wavefronts per block, one block
// per compute unit, block-scaled (1x128 activation scales, 128x128 weight scales) or row/column scaled.
//
// Why.  A compute unit has four SIMDs with one matrix pipe each, and a block of eight wavefronts puts two
// wavefronts on every SIMD.  If both run the same program they leave a barrier together, queue their LDS
// reads together and reach their MFMAs together, so the matrix pipe idles while operands are fetched and
// is fought over afterwards.  Here the two wavefronts of a SIMD run the same program half a K-block
// apart: while one executes its 32 MFMAs (operands already in registers, nothing else to wait for), the
// other reads its operand fragments for the next K-block out of LDS, issues global->LDS loads and, at a
// tile boundary, converts and stores its finished results.  Two block barriers per K-block hand the
// roles over.  The matrix pipe sees an unbroken MFMA stream, and the epilogue of a tile costs nothing
// because it runs under the partner's MFMAs.
//
// Slots.  Group A = wavefronts 0-3, group B = wavefronts 4-7 (one of each per SIMD).  With step T counting
// K-blocks over all tiles a block processes:
//     slot 2T   : A  fetch(T)     B  multiply(T-1)
//     slot 2T+1 : A  multiply(T)  B  fetch(T)
// All global->LDS loads are issued in the fetch phases: a wavefront issues one instruction in about six
// cycles, an MFMA of this shape with its four FMAs fills the 32 cycles the matrix pipe takes, and anything
// else in the multiply phase (a load that waits for the address unit, a branch, scalar bookkeeping) delays
// the MFMAs by that much.  A's wavefronts load the activation tile, B's the weight tile:
//     A, in fetch(T) (slot 2T): activations of stage T+1; waits for them at the end of multiply(T);
//     B, in fetch(T) (slot 2T+1): weights of stage T+2; waits for them at the end of fetch(T+1).
// Every load has more than a whole slot to land, and every wait sits right before a barrier.
//
// LDS.  A stage is 256 x 128 weight bytes plus 256 x 128 activation bytes.  Activation fragments are all
// read in the fetch phases (stage T: slots 2T and 2T+1), so its slot is free for stage T+2 from slot 2T+2 on
// and for A, which loads only one stage ahead, two activation stages suffice.  Weight fragments are also
// read during the multiply phases (stage T: until the end of slot 2T+2); B writes stage T+2 from slot 2T+1
// on, into the slot stage T-1 left at the end of slot 2T: three weight stages.  3 x 32 KB + 2 x 32 KB = 160 KB.
//
// Operand roles and layouts are those of the tile kernel in fp8_gemm.hip (weights in the MFMA A slot,
// XOR-permuted row-major LDS image filled by global_load_lds_dwordx4), with one change: the 128 weight
// rows of a wavefront are dealt to the MFMA tiles so that a 16-byte store instruction writes whole 64-byte
// segments: tile t, A-row i  <->  column (t >> 1) * 32 + (i >> 2) * 8 + (t & 1) * 4 + (i & 3).  Lane group
// lg = i >> 2 then holds eight consecutive columns per pair of tiles, and the four lanes that share an output
// row (16 lanes apart) cover 64 contiguous bytes per store.  The memory side combines the lanes of one store
// instruction, not the instructions: with 32 consecutive columns per lane (four stores of 16 bytes at a
// 64-byte stride) results left at 3.1 TB/s, this way at 6.5 TB/s, and all compute units store at once.  Wavefront
// shares that lie inside the matrix go one step further and pair the rows (store_piece_pair): the lanes of an even
// row and of the odd row after it swap a piece each, and a store instruction writes whole 128-byte lines.
//
// Registers.  Two wavefronts per SIMD leave 256 registers each: 128 fp32 accumulators, the four activation
// fragments of the K-block (32) and a ring of three weight fragments (24) that the multiply phase refills two
// MFMA rows ahead of use.
//
// Short tiles (JN = 1, grouped problems with few rows per segment).  The same program on tiles of 64 rows: each
// wavefront of a group takes one 16-row fragment, 32 accumulators.  The step is then set by how fast a compute unit
// can stream its 32 KB of weights, not by MFMAs on rows that do not exist; the tiles of the last, partly filled
// round of the grid are cut along K so that every compute unit streams to the end (finish_cut_tile).

#include "fp8_gemm_common.h"
#include <mutex>

namespace fg {
namespace {

constexpr int kBM = 256, kBN = 256;
constexpr int kThreads = 512;
constexpr int kWStageBytes = kBN * 128, kXStageBytes = kBM * 128;
constexpr int kWStages = 3, kXStages = 2;  // see "LDS" in the header comment
constexpr int kXRegion = kWStages * kWStageBytes;
constexpr int kLdsBytes = kXRegion + kXStages * kXStageBytes;  // 160 KB, all of a compute unit's LDS
constexpr int kTN = 8, kTM = 4;         // MFMA tiles per wavefront: 128 weight rows x 64 activation rows
// Wave priorities of the phases: the fetch phase is the longer one and every instruction of it sits on the
// path to the barrier that releases the partner's next MFMAs.
constexpr int kFetchPrio = 1, kMultiplyPrio = 0;
constexpr int kSlabsPerWave = 8;        // 1 KB global->LDS loads per wavefront and stage

struct PpArgs {
  GemmArgs g;
  int n_tiles;
  // Stream-K (sk != 0): the n_tiles * KB steps, tile after tile, are cut into gridDim.x contiguous ranges of
  // sk_q or sk_q + 1 steps (the first sk_r ranges get the extra step).  A tile that straddles ranges is
  // finished through the workspace: fp32 partial tiles and one arrival counter per (range, wavefront).
  int sk, sk_q, sk_r;
  // sk_split != 0: every tile is cut into sk_split ranges of sk_q steps (sk_q * sk_split = KB, sk_r = 0, grid =
  // tiles * sk_split), and the blocks of one XCD take the same cut of consecutive tiles: they walk the same K
  // offsets at the same time and share operand panels in their L2, as whole-tile launches do.
  int sk_split;
  // Stream-K over the last n_tiles tiles of a larger problem (the whole rounds before them ran in a launch of their
  // own): tile t of this launch is the tile that whole-tile launches number t + tile_base.
  int tile_base;
  float* partials;
  unsigned int* counters;
  // Start-up delay of block b: (b mod 16) * stagger sleeps of about 1000 cycles.  With short K loops all compute
  // units would finish their tiles together and push 32 MB of results at the memory at once, over and over,
  // each time stalling on the stores for longer than a tile takes to compute; spread over the time the
  // memory needs for one such batch, the stores of one unit overlap the MFMAs of the others.
  int stagger;
  // Grouped problem (groups != nullptr): the rows of X and C are cut into n_groups consecutive segments,
  // segment e ends before row groups[e] (cumulative ends, the `offs` convention of the reference's grouped GEMM,
  // src/flag_gems/ops/scaled_grouped_mm.py:111-114) and is multiplied by weight matrix e (w_group_stride bytes and
  // ws_group_stride floats apart).  Tiles never straddle segments: segment e has ceil(rows_e / 256) tile rows.  The
  // host cannot know the tile count without reading groups back, so it passes an upper bound in n_tiles and
  // g.tiles_m and the kernel derives the real ones.
  const int* groups;
  int n_groups;
  int64_t w_group_stride, ws_group_stride;
  // Grouped problem whose rows are gathered (row_index != nullptr): row m of the sorted order is row
  // row_index[m] / index_div of X and of its scales (the reference's MoE kernel reads its tokens the same way,
  // sorted_token_ids // top_k, src/flag_gems/fused/fused_moe.py:1111); entries are forced into [0, x_rows).
  const int* row_index;
  int index_div, x_rows;
  // the table the loaders gather through: row_index, or null when the rows are already in sorted order and row_index
  // only addresses the scattered result (index_div == 0)
  const int* gather_index;
  // Scattered results (c_rows > 0, with row_index): the result of sorted row m goes to row row_index[m] of C, which
  // has c_rows rows; entries outside [0, c_rows) are padding and store nothing.  With row_weight the fp32 sums are
  // multiplied by row_weight[row_index[m]] before the cast.  This is where and how the reference's MoE kernel
  // writes (offs_token, token_mask, MUL_ROUTED_WEIGHT: src/flag_gems/fused/fused_moe.py:1484-1509).
  int c_rows;
  const float* row_weight;
  // Short tiles of a grouped problem, the last round cut along K (cut_shift > 0): the first cut_full tiles, whole
  // rounds of the grid, are work items of their own; each of the rest is 2^cut_shift work items of cut_steps
  // K-blocks, item cut_full + r = tile cut_full + (r >> cut_shift), cut (r & mask), and the items of a tile add
  // their sums through `partials` and `counters` (finish_cut_tile).  The host passes the largest shift the shape
  // and the workspace allow in cut_shift; the kernel, which knows the real tile count, replaces it by the one it
  // takes and sets cut_full and cut_steps.
  int cut_shift, cut_steps, cut_full;
  uint64_t group4_magic;  // ceil(2^40 / (4 * tiles_n)) when that divides every tile number exactly, else 0 (see tile_of_sid)
};

constexpr int kMaxCutItems = 1024;  // 64 KB slots of partial sums for cut tiles (64 MB): a work item of a 64 JN-row tile takes JN of them
constexpr int kPartialFloatsPerWave = 64 * 128;                      // one wavefront's 64 x 128 results
constexpr int kPartialFloatsPerSlot = 8 * kPartialFloatsPerWave;     // a whole 256 x 256 tile
constexpr size_t kPartialSlotBytes = (size_t)kPartialFloatsPerSlot * 4;  // 256 KB

// Tile number -> (tile row, tile column): four tile rows are walked before moving along N.  The division by
// 4 * tiles_n is a multiplication by a constant the host prepares (`magic` = ceil(2^40 / (4 * tiles_n)), exact while
// tiles * 4 * tiles_n < 2^40; 0 = divide): a walk crosses a tile boundary once per K / 128 steps, in a phase with
// little slack, and a 32-bit division by a run-time value costs about a thousand cycles there.
__device__ __forceinline__ void tile_of_sid(int sid, int tiles_m, int tiles_n, uint64_t magic, int& tm, int& tn) {
  constexpr int GROUP_M = 4;
  const int per_group = GROUP_M * tiles_n;
  const int g = magic != 0 ? (int)(((uint64_t)(uint32_t)sid * magic) >> 40) : sid / per_group;
  const int first_m = g * GROUP_M;
  const int gm = (tiles_m - first_m < GROUP_M) ? tiles_m - first_m : GROUP_M;
  const uint32_t r = (uint32_t)(sid - g * per_group);
  uint32_t q;  // r / gm
  if (gm == 4) q = r >> 2;
  else if (gm == 3) q = r / 3u;
  else if (gm == 2) q = r >> 1;
  else q = r;
  tm = first_m + (int)(r - q * (uint32_t)gm);
  tn = (int)q;
}

// Same XCD-aware order as the tile kernel: ids congruent mod 8 (one XCD) walk a contiguous run of tiles,
// four tile rows at a time.
__device__ __forceinline__ void tile_of_index(int vid, int tiles_m, int tiles_n, uint64_t magic, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  const int xcd = vid & 7, local = vid >> 3;
  const int base = total >> 3, rem = total & 7;
  const int sid = xcd * base + (xcd < rem ? xcd : rem) + local;
  tile_of_sid(sid, tiles_m, tiles_n, magic, tm, tn);
}

// A block visits the virtual ids blockIdx.x, blockIdx.x + gridDim.x, ...  The grid is either the tile count
// (one round) or the number of compute units, a multiple of 8, so a block stays on its XCD's run of tiles.
// tile_of_index maps [0, n_tiles) onto the tiles one-to-one.

// weight row (within the wavefront's 128) held by LDS row rho of the wavefront's region
__device__ __forceinline__ int weight_row_of_lds_row(int rho) {
  const int t = rho >> 4, i = rho & 15;
  return (t >> 1) * 32 + (i >> 2) * 8 + (t & 1) * 4 + (i & 3);
}
// first of the eight consecutive output columns that lane group lg holds in MFMA tiles 2q and 2q+1
__device__ __forceinline__ int piece_column(int n_base, int q, int lg) { return n_base + q * 32 + lg * 8; }

// Uniform (scalar) walk over the (tile, K-block) steps of this block, in processing order.  Three of these
// run at different distances: the step being multiplied, the step whose scales are being fetched (one
// ahead) and the stage being loaded (one or two ahead).  A tile change costs two integer divisions and
// happens once per K / 128 steps; everything else per step is an add.
// End of segment e of a grouped problem (uniform, a scalar load), forced into [begin, M]: a table that is not
// ascending or runs past the rows must not send loads or stores outside the operands.
__device__ __forceinline__ int segment_end(const PpArgs& a, int e, int begin) {
  int end = ((const __attribute__((address_space(4))) int*)a.groups)[e];
  end = end < a.g.M ? end : a.g.M;
  return end > begin ? end : begin;
}

// TILE_ROWS: activation rows per tile (kBM; less for the grouped kernel that serves short segments)
// CUTS: the ids are work items of a grouped problem whose tiles are cut along K (PpArgs::cut_shift).
template <bool GROUPED, int TILE_ROWS = kBM, bool CUTS = false>
struct WalkT {
  int idx, kb, m0, n0;  // idx: virtual id (data-parallel rounds) or tile number (stream-K)
  int kb_end;           // the walk leaves the tile (the work item) before this K-block
  int m_end, group;     // first row past the tile's segment (M when the problem is not grouped); its weight matrix
  int n_tiles, tiles_m; // of the whole problem (a grouped problem's are counted by the kernel)
  __device__ __forceinline__ bool inside(const PpArgs& a) const {
    return (CUTS && idx >= a.cut_full ? a.cut_full + ((idx - a.cut_full) >> a.cut_shift) : idx) < n_tiles;
  }
  __device__ __forceinline__ void locate(const PpArgs& a) {
    int tm = 0, tn = 0;
    kb_end = a.g.KB;
    if (CUTS) {
      int tile = idx;
      if (idx >= a.cut_full) {
        const int r = idx - a.cut_full;
        tile = a.cut_full + (r >> a.cut_shift);
        kb = (r - ((r >> a.cut_shift) << a.cut_shift)) * a.cut_steps;
        kb_end = kb + a.cut_steps;
      }
      if (tile < n_tiles) tile_of_index(tile, tiles_m, a.g.tiles_n, a.group4_magic, tm, tn);
    } else if (idx < n_tiles) {
      if (a.sk && a.tile_base == 0) tile_of_sid(idx, tiles_m, a.g.tiles_n, a.group4_magic, tm, tn);
      else if (a.sk) tile_of_index(idx + a.tile_base, tiles_m, a.g.tiles_n, a.group4_magic, tm, tn);
      else tile_of_index(idx, tiles_m, a.g.tiles_n, a.group4_magic, tm, tn);
    }
    m0 = tm * TILE_ROWS; n0 = tn * kBN;
    m_end = a.g.M; group = 0;
    if (GROUPED) {
      // tile row tm of the whole problem -> segment and tile row inside it
      int begin = 0, t = tm, e = 0, end = 0;
      for (; e < a.n_groups; ++e) {
        end = segment_end(a, e, begin);
        const int nt = (end - begin + TILE_ROWS - 1) / TILE_ROWS;
        if (t < nt) break;
        t -= nt;
        begin = end;
      }
      m0 = begin + t * TILE_ROWS; m_end = end; group = e < a.n_groups ? e : 0;
    }
  }
  __device__ __forceinline__ void start(const PpArgs& a, int first_idx, int first_kb, int n_tiles_, int tiles_m_) {
    idx = first_idx; kb = first_kb; n_tiles = n_tiles_; tiles_m = tiles_m_;
    locate(a);
  }
  // true when the walk entered a new tile
  __device__ __forceinline__ bool next(const PpArgs& a) {
    if (++kb < kb_end) return false;
    kb = 0; idx += a.sk ? 1 : (int)gridDim.x;
    locate(a);
    return true;
  }
};

// This wavefront's share of the global->LDS loads of one stage: 8 slabs (1 KB, 8 LDS rows each) of one
// operand tile.  The four wavefronts of group A load the activation tile, those of group B the weight
// tile: the groups run half a step apart and each operand has a moment of its own when an LDS slot is
// free for it (see the main loop).  Per-lane byte offsets are relative to the tile's first row.
struct LoadShare {
  uint32_t off[kSlabsPerWave];
  const uint8_t* ptr;  // uniform: first row of the tile, K-block being loaded

  // valid: rows of the tile inside the matrix; rows past the edge re-read the last row and are never stored
  __device__ __forceinline__ void set_offsets(const GemmArgs& a, int valid, int wave, int lane) {
    const bool weights = wave >= 4;
    const uint32_t ld = (uint32_t)(weights ? a.ldw : a.ldx);
#pragma unroll
    for (int j = 0; j < kSlabsPerWave; ++j) {
      const int slab = (wave & 3) + j * 4;
      const int r = slab * 8 + (lane >> 3);  // LDS row
      const uint32_t chunk = (uint32_t)(((lane & 7) ^ (r & 7)) << 4);
      int row = weights ? (r & 128) + weight_row_of_lds_row(r & 127) : r;
      row = row < valid ? row : valid - 1;
      off[j] = __umul24((uint32_t)row, ld) + chunk;  // row < 256, ld < 2^23 (checked by the host)
    }
  }
  // Activation rows read through an index: offsets are relative to the first row of X (the host checks that
  // x_rows * ldx fits 32 bits); rows past the segment's end repeat its last row, as above.
  __device__ __forceinline__ void set_gathered(const GemmArgs& a, const int* row_index, int index_div, int x_rows,
                                               int m0, int valid, int lane, int wave) {
    const uint32_t ld = (uint32_t)a.ldx;
#pragma unroll
    for (int j = 0; j < kSlabsPerWave; ++j) {
      const int slab = (wave & 3) + j * 4;
      const int r = slab * 8 + (lane >> 3);  // LDS row
      const uint32_t chunk = (uint32_t)(((lane & 7) ^ (r & 7)) << 4);
      const int row = r < valid ? r : valid - 1;
      int src = row_index[m0 + row] / index_div;
      src = src < 0 ? 0 : (src < x_rows ? src : x_rows - 1);
      off[j] = (uint32_t)src * ld + chunk;
    }
    ptr = a.X;
  }
  __device__ __forceinline__ void set_ptr(const GemmArgs& a, int m0, int n0, int wave, int64_t w_group_off = 0) {
    ptr = wave >= 4 ? a.W + w_group_off + (int64_t)n0 * a.ldw : a.X + (int64_t)m0 * a.ldx;
  }
  // m_end: first row past the segment the tile belongs to (M when the problem is not grouped)
  template <int TILE_ROWS = kBM>
  __device__ __forceinline__ void set_tile(const GemmArgs& a, int m0, int n0, int wave, int lane, int m_end, int64_t w_group_off = 0) {
    set_ptr(a, m0, n0, wave, w_group_off);
    const int valid = wave >= 4 ? a.N - n0 : m_end - m0;
    const int most = wave >= 4 ? kBN : TILE_ROWS;
    set_offsets(a, valid < most ? valid : most, wave, lane);
  }
  // The load is written out instead of using the compiler's builtin: the compiler books a global->LDS
  // load as an access that may return through either counter, and from then on turns every wait for an LDS
  // read into lgkmcnt(0), which makes the multiply phase wait for fragments it needs two rows later.
  // stage_lds: LDS byte address of this wavefront's first slab in the stage (uniform).
  __device__ __forceinline__ void issue_one(uint32_t stage_lds, int q) const {
    asm volatile("s_add_u32 m0, %2, %3\n\t"
                 "s_nop 0\n\t"
                 "global_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(off[q]), "s"(ptr), "s"(stage_lds), "n"(q * 4 * 1024)
                 : "memory", "m0", "scc");
  }
};

__device__ __forceinline__ int fragment_offset(int lane) {
  const int r = lane & 15, g = lane >> 4;
  return r * 128 + ((g ^ (r & 7)) << 4);
}

__device__ __forceinline__ v8i read_frag(const uint8_t* region, int rg, int lane_off) {
  const u32x4 lo = *reinterpret_cast<const u32x4*>(region + rg * 2048 + lane_off);
  const u32x4 hi = *reinterpret_cast<const u32x4*>(region + rg * 2048 + (lane_off ^ 64));
  v8i f;
  f[0] = (int)lo.x; f[1] = (int)lo.y; f[2] = (int)lo.z; f[3] = (int)lo.w;
  f[4] = (int)hi.x; f[5] = (int)hi.y; f[6] = (int)hi.z; f[7] = (int)hi.w;
  return f;
}

// MFMA with a zero accumulator input, result in architectural VGPRs
__device__ __forceinline__ v4f mfma_partial(const v8i& w, const v8i& x) {
  v4f p = {};
  asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=&v"(p) : "v"(w), "v"(x));
  return p;
}

__device__ __forceinline__ void mfma_accumulate(v4f& c, const v8i& w, const v8i& x) {
  asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+v"(c) : "v"(w), "v"(x));
}

// int8 operands (kModeRowColI8): the same fragment as two 16x16x64 products (`half` = 0: the lane's first 16 bytes of
// the K-block, 1: its second 16), int32 sums kept as bit patterns in the accumulator registers; the two instructions
// take as long as the one fp8 instruction.  The multiply phase issues the two halves of one accumulator kTM
// instructions apart, so that the matrix pipe never waits for the sum it has just started.
// bf16 and fp16 operands (kModeRowColBF16 / F16) take the same route: a lane's 16 bytes are eight elements, the
// fragment two 16x16x32 products into fp32 sums, and the pair again takes as long as the one fp8 instruction.
template <int MODE>
__device__ __forceinline__ void mfma_accumulate_half(v4f& c, const v8i& w, const v8i& x, int half) {
  typedef int v4i_ __attribute__((ext_vector_type(4)));
  const v4i_ wh = half ? v4i_{w[4], w[5], w[6], w[7]} : v4i_{w[0], w[1], w[2], w[3]};
  const v4i_ xh = half ? v4i_{x[4], x[5], x[6], x[7]} : v4i_{x[0], x[1], x[2], x[3]};
  if constexpr (MODE == kModeRowColBF16) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(wh), "v"(xh));
  else if constexpr (MODE == kModeRowColF16) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(wh), "v"(xh));
  else asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(c) : "v"(wh), "v"(xh));
}

// Scales that are powers of two (POW2): the block-scaled form of the instruction multiplies the products by
// 2^(sw - 127) * 2^(sx - 127) on their way into the sum, so the matrix pipe accumulates the scaled K-blocks itself and
// the multiply phase has no vector-ALU work at all.  sw / sx: E8M0 exponent in the low byte of a register per lane,
// taken for the operand row the lane holds (lane & 15); every 32-element K group of a row gets the same one here.
__device__ __forceinline__ void mfma_scaled_accumulate(v4f& c, const v8i& w, const v8i& x, int sw, int sx) {
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[0,0,0] op_sel_hi:[0,0,0]"
               : "+v"(c)
               : "v"(w), "v"(x), "v"(sw), "v"(sx));
}
__device__ __forceinline__ int e8m0_of(float s) { return (int)((float_to_bits(s) >> 23) & 0xFFu); }

// acc += p * s.  A wavefront issues one instruction every four cycles and the matrix pipe takes an MFMA of
// this shape every 32, so a multiply step has eight issue slots: the MFMA, these four FMAs and three spare
// (LDS reads, tile loads).  p is the result of the MFMA issued TWO steps earlier: at least 64 cycles have
// passed since its issue, more than the 11 wait states (44 cycles) gfx950 requires between an 8-pass MFMA
// write and a VALU read, so no s_nop is spent in the steady state.  NOPS > 0 pads the tail of the phase.
template <int NOPS>
__device__ __forceinline__ void scale_into(v4f& acc, const v4f& p, float s) {
  float a0 = acc[0], a1 = acc[1], a2 = acc[2], a3 = acc[3];
  if (NOPS > 0) {
    asm volatile("s_nop %9\n\t"
                 "v_fmac_f32 %0, %4, %8\n\t"
                 "v_fmac_f32 %1, %5, %8\n\t"
                 "v_fmac_f32 %2, %6, %8\n\t"
                 "v_fmac_f32 %3, %7, %8"
                 : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3)
                 : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(s), "n"(NOPS - 1));
  } else {
    asm volatile("v_fmac_f32 %0, %4, %8\n\t"
                 "v_fmac_f32 %1, %5, %8\n\t"
                 "v_fmac_f32 %2, %6, %8\n\t"
                 "v_fmac_f32 %3, %7, %8"
                 : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3)
                 : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(s));
  }
  acc[0] = a0; acc[1] = a1; acc[2] = a2; acc[3] = a3;
}

// Activation scales are fetched one step ahead with loads the compiler does not track, and picked up after an
// explicit count.  Left to the compiler, the wait for these four values becomes vmcnt(0) in the middle of a
// slot, which also waits for the tile loads issued after them.  The destination is an in/out operand so that
// the value keeps one register across loop iterations.
__device__ __forceinline__ void load_f32_untracked(float& v, uint32_t byte_off, const float* base) {
  asm volatile("global_load_dword %0, %1, %2" : "+v"(v) : "v"(byte_off), "s"(base) : "memory");
}
// cur = nxt once at most PENDING younger vector-memory operations are outstanding
template <int PENDING>
__device__ __forceinline__ void wait_and_take(float (&cur)[kTM], const float (&nxt)[kTM]) {
  static_assert(kTM == 4, "four activation fragments per wavefront");
  asm volatile("s_waitcnt vmcnt(%8)\n\t"
               "v_mov_b32 %0, %4\n\t"
               "v_mov_b32 %1, %5\n\t"
               "v_mov_b32 %2, %6\n\t"
               "v_mov_b32 %3, %7"
               : "=&v"(cur[0]), "=&v"(cur[1]), "=&v"(cur[2]), "=&v"(cur[3])
               : "v"(nxt[0]), "v"(nxt[1]), "v"(nxt[2]), "v"(nxt[3]), "n"(PENDING)
               : "memory");
}
template <int PENDING>
__device__ __forceinline__ void wait_vmem() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(PENDING) : "memory");
}

// 16 bytes of results
__device__ __forceinline__ void store_result_16(uint16_t* p, u32x4 v) {
  *reinterpret_cast<u32x4*>(p) = v;
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const bf16x2_t h = __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t);
  return __builtin_bit_cast(uint32_t, h);
}
// Two results as the 16-bit output type, F16: fp16, else bf16 (round to nearest even both).  The empty statement
// keeps the compiler from folding a multiplication that produced the value into the conversion (one rounding
// instead of the two that the tile kernels and the reference perform).
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
template <bool F16>
__device__ __forceinline__ uint32_t pack_out(float lo, float hi) {
  if (!F16) return pack_bf16(lo, hi);
  asm volatile("" : "+v"(lo), "+v"(hi));
  const f16x2_t h = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, h);
}
// the two halves of such a word as fp32
template <bool F16>
__device__ __forceinline__ float unpack_lo(uint32_t w) {
  return F16 ? (float)__builtin_bit_cast(f16x2_t, w)[0] : bits_to_float(w << 16);
}
template <bool F16>
__device__ __forceinline__ float unpack_hi(uint32_t w) {
  return F16 ? (float)__builtin_bit_cast(f16x2_t, w)[1] : bits_to_float(w & 0xFFFF0000u);
}

// The value that the lane holding the neighbouring row (l16 ^ 1, same lg: the adjacent lane) has in `v`.
__device__ __forceinline__ uint32_t from_row_neighbour(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1 /* quad_perm [1, 0, 3, 2] */, 0xF, 0xF, true);
}
// Two pieces that are neighbours in a row (64 + 64 bytes: `lo` the lower columns) leave as whole 128-byte runs: the
// lanes of an even row and of the odd row after it exchange one piece each, after which the eight lanes of such a pair
// of rows hold the 128 bytes of the even row (first store) and of the odd row (second store).  A store instruction
// then touches 8 memory lines instead of 16 halves, and the time a compute unit's address unit spends on a store
// goes with the lines it touches: measured on whole launches at M = 4096, N = 32768, K = 512: 103 -> 92 us;
// N = 24576, K = 1536: 160 -> 150 us; N = 7168, K = 2304: 74 -> 69 us.
// `even_row`: the lane's position in the even row of its pair, at the columns of `lo` (odd lanes: of `hi`).
__device__ __forceinline__ void store_piece_pair(uint16_t* even_row, int64_t ldc, bool odd, const uint32_t (&lo)[4], const uint32_t (&hi)[4]) {
  u32x4 first, second;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t lo_there = from_row_neighbour(lo[e]), hi_there = from_row_neighbour(hi[e]);
    first[e] = odd ? hi_there : lo[e];
    second[e] = odd ? hi[e] : lo_there;
  }
  store_result_16(even_row, first);
  store_result_16(even_row + ldc, second);
}

// Stores the wavefront's 64 x 128 results as bf16.  Lane (l16, lg) holds, for every activation tile j, four
// pieces of eight consecutive columns of row m_base + 16 j + l16: piece q starts at column
// n_base + 32 q + 8 lg and comes from MFMA tiles 2q and 2q+1.  The host guarantees ldc % 8 == 0 and a 16-byte
// aligned C, so a piece leaves as one 16-byte store, and the four lanes of a row cover 64 contiguous bytes per
// store instruction (tiles with edges), or pairs of pieces leave as whole 128-byte runs (ALIGNED: store_piece_pair).
// Row/column mode: the sums are scaled by a_scale[m] * b_scale[n] first, and the bias is added to the rounded
// value, in bf16, as the reference's epilogue does (src/flag_gems/fused/cutlass_scaled_mm.py:288-305).
// ALIGNED: the tile lies inside the matrix; a wavefront then issues exactly kStoresPerTile store instructions.
constexpr int kStoresPerTile = 16;
// SCATTER (grouped problems): rows go where out_index says (see PpArgs::c_rows).
// JN: activation fragments per wavefront (rows m_base .. m_base + 16 JN).
// F16: the results are fp16 (else bf16).
// NT, q0: `acc` holds the NT MFMA tiles of pieces q0 .. q0 + NT / 2 - 1 (all eight, or the half that the finish of a
// shared tile sums at a time).
template <int MODE, bool ALIGNED, bool SCATTER = false, int JN = kTM, bool F16 = false, int NT = kTN>
__device__ __forceinline__ void store_tile(const GemmArgs& a, const v4f (&acc)[NT][JN], int m_base, int n_base,
                                           int l16, int lg, int m_end, const int* out_index = nullptr, int c_rows = 0,
                                           const float* row_weight = nullptr, int q0 = 0) {
  if constexpr (!ALIGNED && !SCATTER && NT % 4 == 0 && MODE == kModeBlock) {
    // a wavefront's share that lies inside the matrix (uniform) takes the stores of whole tiles (block scales only:
    // the row/column modes' instantiations with edges have no registers left for a second store path and spill)
    if (m_base + 16 * JN <= m_end && piece_column(n_base, q0 + NT / 2, 0) <= a.N) {
      store_tile<MODE, true, false, JN, F16, NT>(a, acc, m_base, n_base, l16, lg, m_end, nullptr, 0, nullptr, q0);
      return;
    }
  }
  constexpr bool kPairs = ALIGNED && !SCATTER && NT % 4 == 0;  // whole tiles: pieces leave two at a time
  const bool odd = (l16 & 1) != 0;
  if (MODE != kModeBlock) {
    uint32_t kept[JN][4];  // kPairs: the lower piece of the pair, while the upper one is computed
    (void)kept;
    // eight columns at a time, so that only eight column scales and bias values are live
#pragma unroll
    for (int q = 0; q < NT / 2; ++q) {
      const int n = piece_column(n_base, q0 + q, lg);
      const bool full = ALIGNED || n + 8 <= a.N;
      float sb[8], bias[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int ne = n + e < a.N ? n + e : a.N - 1;
        sb[e] = a.ws[a.ws_per_col ? ne : 0];
        bias[e] = a.bias ? load_as_float(a.bias, ne, a.bias_dtype) : 0.f;
      }
#pragma unroll
      for (int j = 0; j < JN; ++j) {
        const int m = m_base + j * 16 + l16;
        if (!ALIGNED && m >= m_end) continue;
        const float sa = a.xs[a.xs_per_row ? m : 0];
        uint32_t w[4];
#pragma unroll
        for (int h = 0; h < 4; ++h) {  // two columns per word
          const int t = 2 * q + (h >> 1), e0 = (h & 1) * 2;
          // (int8 operands: the registers hold int32 sums.  The element is copied to a scalar before the bit cast:
          // a bit cast applied to the vector element itself reads element 0 whatever the index.)
          const float r0 = acc[t][j][e0], r1 = acc[t][j][e0 + 1];
          const float s0 = MODE == kModeRowColI8 ? (float)__float_as_int(r0) : r0;
          const float s1 = MODE == kModeRowColI8 ? (float)__float_as_int(r1) : r1;
          float v0 = (s0 * sa) * sb[4 * (h >> 1) + e0];
          float v1 = (s1 * sa) * sb[4 * (h >> 1) + e0 + 1];
          if (MODE >= kModeRowColBF16) {  // one rounding, the bias before it
            if (a.bias) { v0 = v0 + bias[4 * (h >> 1) + e0]; v1 = v1 + bias[4 * (h >> 1) + e0 + 1]; }
            w[h] = pack_out<F16>(v0, v1);
            continue;
          }
          w[h] = pack_out<F16>(v0, v1);
          if (a.bias)
            w[h] = pack_out<F16>(unpack_lo<F16>(w[h]) + bias[4 * (h >> 1) + e0],
                                 unpack_hi<F16>(w[h]) + bias[4 * (h >> 1) + e0 + 1]);
        }
        if constexpr (kPairs) {
          if ((q & 1) == 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e) kept[j][e] = w[e];
          } else {
            // (q0 + q is odd: this lane's columns of the lower piece start 32 columns before n)
            store_piece_pair(reinterpret_cast<uint16_t*>(a.C) + (int64_t)(m - (l16 & 1)) * a.ldc + n - 32 + (l16 & 1) * 32,
                             a.ldc, odd, kept[j], w);
          }
          continue;
        }
        uint16_t* const cp = reinterpret_cast<uint16_t*>(a.C) + (int64_t)m * a.ldc + n;
        if (full) {
          *reinterpret_cast<u32x4*>(cp) = u32x4{w[0], w[1], w[2], w[3]};
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n + e < a.N) cp[e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
        }
      }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < JN; ++j) {
    const int m = m_base + j * 16 + l16;
    if (!ALIGNED && m >= m_end) continue;
    int64_t out_row = m;
    float wgt = 1.f;
    if (SCATTER && out_index != nullptr) {
      const int idx = out_index[m];
      if (idx < 0 || idx >= c_rows) continue;
      out_row = idx;
      if (row_weight != nullptr) wgt = row_weight[idx];
    }
    uint16_t* const row = reinterpret_cast<uint16_t*>(a.C) + out_row * a.ldc;
    uint32_t w[2 * NT];
    if (SCATTER && row_weight != nullptr) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        w[2 * t] = pack_out<F16>(acc[t][j][0] * wgt, acc[t][j][1] * wgt);
        w[2 * t + 1] = pack_out<F16>(acc[t][j][2] * wgt, acc[t][j][3] * wgt);
      }
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        w[2 * t] = pack_out<F16>(acc[t][j][0], acc[t][j][1]);
        w[2 * t + 1] = pack_out<F16>(acc[t][j][2], acc[t][j][3]);
      }
    }
    if constexpr (kPairs) {
#pragma unroll
      for (int q = 0; q < NT / 2; q += 2) {
        const uint32_t lo[4] = {w[4 * q], w[4 * q + 1], w[4 * q + 2], w[4 * q + 3]};
        const uint32_t hi[4] = {w[4 * q + 4], w[4 * q + 5], w[4 * q + 6], w[4 * q + 7]};
        store_piece_pair(reinterpret_cast<uint16_t*>(a.C) + (int64_t)(m - (l16 & 1)) * a.ldc + piece_column(n_base, q0 + q, lg) + (l16 & 1) * 32,
                         a.ldc, odd, lo, hi);
      }
      continue;
    }
#pragma unroll
    for (int q = 0; q < NT / 2; ++q) {
      const int n = piece_column(n_base, q0 + q, lg);
      if (ALIGNED || n + 8 <= a.N) {
        store_result_16(row + n, u32x4{w[4 * q], w[4 * q + 1], w[4 * q + 2], w[4 * q + 3]});
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (n + e < a.N) row[n + e] = (uint16_t)(w[4 * q + (e >> 1)] >> (16 * (e & 1)));
      }
    }
  }
}

// Range arithmetic of the stream-K split (all uniform).
__device__ __forceinline__ int sk_range_begin(const PpArgs& a, int pos) {
  return pos * a.sk_q + (pos < a.sk_r ? pos : a.sk_r);
}
__device__ __forceinline__ int sk_range_of_step(const PpArgs& a, int step) {
  const int big = a.sk_r * (a.sk_q + 1);
  return step < big ? step / (a.sk_q + 1) : a.sk_r + (step - big) / a.sk_q;
}

// Finishes a tile that this block computed only part of.  Each wavefront handles its own 64 x 128 piece:
// it publishes its partial sums, then counts itself in; the wavefront that arrives last (of the ranges that
// share the tile) adds all partial sums in range order -- the same order whoever comes last, so the
// result does not depend on timing -- stores the piece, and resets the counter for the next launch.
// Nobody waits for anybody.  On entry and exit no vector-memory operation of this wavefront is pending.
template <int MODE, bool F16>
__device__ __forceinline__ void finish_partial_tile(const PpArgs& a, const v4f (&acc)[kTN][kTM], int tile, int pos,
                                                    int m_base, int n_base, int wave, int lane, int l16, int lg) {
  const int s_lo = tile * a.g.KB;
  const int first = sk_range_of_step(a, s_lo), last = sk_range_of_step(a, s_lo + a.g.KB - 1);
  const int nseg = last - first + 1;
  // a range owns two slots: [0] for the tile its range starts in, [1] for the tile it ends in when that is
  // another one
  auto slot_of = [&](int q) __attribute__((always_inline)) -> float* {
    const int which = (sk_range_begin(a, q) >= s_lo) ? 0 : 1;
    return a.partials + ((size_t)(q * 2 + which) * 8 + wave) * kPartialFloatsPerWave;
  };
  const uint32_t lane_off = (uint32_t)lane * 16u;
  float* const mine = uniform_ptr(slot_of(pos));
#pragma unroll
  for (int t = 0; t < kTN; ++t)
#pragma unroll
    for (int j = 0; j < kTM; ++j) store_x4_agent(mine + (t * kTM + j) * 256, lane_off, acc[t][j]);
  wait_vmem<0>();
  unsigned int* const cnt = a.counters + first * 8 + wave;
  unsigned int prev = 0;
  if (lane == 0) prev = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  prev = (unsigned int)__builtin_amdgcn_readfirstlane((int)prev);
  if (prev != (unsigned int)(nseg - 1)) return;
  // Last to arrive.  Its own sums are in the workspace like everybody's, so the accumulators are free:
  // half of the piece (16 columns per lane and row) is summed at a time, every range's loads in flight together
  // with the running sum.
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    v4f r[kTN / 2][kTM];
    for (int q = first; q <= last; ++q) {
      const float* const src = uniform_ptr(slot_of(q));
      v4f tmp[kTN / 2][kTM];
#pragma unroll
      for (int t = 0; t < kTN / 2; ++t)
#pragma unroll
        for (int j = 0; j < kTM; ++j) load_x4_agent(tmp[t][j], src + ((half * (kTN / 2) + t) * kTM + j) * 256, lane_off);
#pragma unroll
      for (int t = 0; t < kTN / 2; ++t)  // the values are operands of the wait, so no use can move above it
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(tmp[t][0]), "+v"(tmp[t][1]), "+v"(tmp[t][2]), "+v"(tmp[t][3]) : : "memory");
#pragma unroll
      for (int t = 0; t < kTN / 2; ++t)
#pragma unroll
        for (int j = 0; j < kTM; ++j) {
          // plain assignment for the first range keeps "0 + x" out of the sum; int8 operands: int32 sums, added as such
          if (q == first) r[t][j] = tmp[t][j];
          else if (MODE == kModeRowColI8) r[t][j] = __builtin_bit_cast(v4f, __builtin_bit_cast(v4i, r[t][j]) + __builtin_bit_cast(v4i, tmp[t][j]));
          else r[t][j] += tmp[t][j];
        }
    }
    // (scales and bias of the row/column modes, conversion, 16-byte stores or single elements at the ragged edge)
    store_tile<MODE, false, false, kTM, F16, kTN / 2>(a.g, r, m_base, n_base, l16, lg, a.g.M, nullptr, 0, nullptr, half * 2);
  }
  if (lane == 0) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the counted waits of the main loop start from zero
}

// Finishes a short tile of a grouped problem that is cut along K (PpArgs::cut_shift): the same protocol as
// finish_partial_tile -- publish, count in, the last of the tile's work items to arrive adds all partial sums in cut
// order and stores -- on the wavefront's 16 JN x 128 piece, which is small enough to be summed whole and handed to
// store_tile, so gathered, scattered and weighted results take the one store path.  A slot per (work item, wavefront).
template <bool SCATTER, int JN, bool F16>
__device__ __forceinline__ void finish_cut_tile(const PpArgs& a, const v4f (&acc)[kTN][JN], int item, int m_base, int n_base,
                                                int m_end, int wave, int lane, int l16, int lg) {
  constexpr int kFloats = kTN * JN * 256;  // per wavefront
  // item, tile: counted from the first cut one
  const int tile = item >> a.cut_shift, cuts = 1 << a.cut_shift;
  const uint32_t lane_off = (uint32_t)lane * 16u;
  float* const mine = uniform_ptr(a.partials + ((size_t)item * 8 + wave) * kFloats);
#pragma unroll
  for (int t = 0; t < kTN; ++t)
#pragma unroll
    for (int j = 0; j < JN; ++j) store_x4_agent(mine + (t * JN + j) * 256, lane_off, acc[t][j]);
  wait_vmem<0>();
  unsigned int* const cnt = a.counters + tile * 8 + wave;
  unsigned int prev = 0;
  if (lane == 0) prev = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  prev = (unsigned int)__builtin_amdgcn_readfirstlane((int)prev);
  if (prev != (unsigned int)(cuts - 1)) return;
  // A part of the piece at a time (its own sums are in the workspace like everybody's, so the accumulators are free):
  // halves for short tiles, quarters for 256-row tiles; sixteen registers of partial sums in flight.
  constexpr int kParts = JN == kTM ? 4 : 2;   // parts of the piece
  constexpr int kNT = kTN / kParts;           // MFMA tiles per part
  constexpr int kBatch = 4 / JN;              // MFMA tiles per load batch
#pragma unroll
  for (int part = 0; part < kParts; ++part) {
    v4f r[kNT][JN];
    for (int q = 0; q < cuts; ++q) {
      const float* const src = uniform_ptr(a.partials + ((size_t)((tile << a.cut_shift) + q) * 8 + wave) * kFloats);
#pragma unroll
      for (int b = 0; b < kNT / kBatch; ++b) {
        v4f tmp[kBatch][JN];
#pragma unroll
        for (int t = 0; t < kBatch; ++t)
#pragma unroll
          for (int j = 0; j < JN; ++j)
            load_x4_agent(tmp[t][j], src + ((part * kNT + b * kBatch + t) * JN + j) * 256, lane_off);
#pragma unroll
        for (int t = 0; t < kBatch; ++t)
#pragma unroll
          for (int j = 0; j < JN; ++j)  // the values are operands of the wait, so no use can move above it
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(tmp[t][j]) : : "memory");
#pragma unroll
        for (int t = 0; t < kBatch; ++t)
#pragma unroll
          for (int j = 0; j < JN; ++j) {
            const int tt = b * kBatch + t;
            if (q == 0) r[tt][j] = tmp[t][j]; else r[tt][j] += tmp[t][j];  // (no "0 + x" in the sum)
          }
      }
    }
    store_tile<kModeBlock, false, SCATTER, JN, F16, kNT>(a.g, r, m_base, n_base, l16, lg, m_end,
                                                         SCATTER && a.c_rows > 0 ? a.row_index : nullptr, a.c_rows,
                                                         a.row_weight, part * (kNT / 2));
  }
  if (lane == 0) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the counted waits of the main loop start from zero
}

// ALIGNED: M and N are multiples of the tile; no tile has an edge, and the per-lane offsets of the tile loads
// and of the scale loads never change (a tile change then touches scalar registers only).
// GROUPED: the rows are segments with a weight matrix each (see PpArgs::groups).
// POW2: block scales that are powers of two, applied by the instruction (mfma_scaled_accumulate).
// JN: activation fragments (16 rows) per wavefront; the tile has 64 JN rows.  Less than kTM only for grouped problems
// whose segments are short: a 256-row tile costs its 256 rows of MFMAs however few of them belong to the segment, and
// that, not the weight stream, sets the time of a step when a tile holds a few dozen rows.  With JN = 1 the four
// wavefronts of a group take 16 rows each, the activation image in LDS keeps its 256-row layout (the rows past the
// 64th are loaded like rows past an edge and never read), and everything else runs unchanged.
// F16: the results are fp16 (else bf16).  A template parameter and not a test of c_dtype in the flush: with both
// forms of the stores in one kernel the bf16 flush of short-K problems got 5 % slower.
template <bool SK, int MODE, bool ALIGNED, bool GROUPED = false, bool POW2 = false, int JN = kTM, bool F16 = false>
__global__ __launch_bounds__(kThreads) void fp8_gemm_pingpong_kernel(PpArgs a) {
  static_assert(JN == kTM || (GROUPED && JN >= 1 && JN < kTM), "short tiles: grouped problems only");
  constexpr int kTileRows = 64 * JN;
  constexpr bool kDeferTail = JN == kTM;  // the FMAs of a step's last two MFMAs run after the barrier that ends the slot
  constexpr bool kCuts = GROUPED;  // tiles may be cut along K (cut_shift = 0: they are not)
  // Short tiles finish a cut tile in the fetch slot that follows it, like a whole tile.  With 128 accumulators that
  // code does not fit the registers of the hot loop (242 spilled), and the walk of a block is [whole tiles][its cut
  // work items] anyway: the loop runs once for the whole tiles and once per work item, which is finished between
  // the runs, as the shared tiles of a stream-K launch are.
  constexpr bool kCutsInLoop = kCuts && JN < kTM;
  // Short tiles stream weights for next to no arithmetic, and what sets their pace is how many weight bytes a compute
  // unit has in flight: the activation stages shrink to the tile's rows and the LDS they leave holds a fourth weight
  // stage, so that group B loads three steps ahead instead of two.
  constexpr int kWSt = JN < kTM ? kWStages + 1 : kWStages;
  constexpr int kXStBytes = JN < kTM ? kTileRows * 128 : kXStageBytes;
  constexpr int kXReg = kWSt * kWStageBytes;
  static_assert(kXReg + kXStages * kXStBytes <= kLdsBytes, "LDS");
  static_assert(!POW2 || (MODE == kModeBlock && !GROUPED), "power-of-two scales: plain block-scaled problems");
  static_assert(!GROUPED || (!SK && !ALIGNED && MODE == kModeBlock), "grouped problems: whole tiles with edges, block scales");
  using Walk = WalkT<GROUPED, kTileRows, kCuts>;
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const GemmArgs& g = a.g;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2;       // 0: group A, 1: group B
  const int wave_m = wave & 3;     // quarter of the activation tile (64 rows of 256)
  const int wm0 = wave_m * 16 * JN, wn0 = grp * 128;
  const int l16 = lane & 15, lg = lane >> 4;
  const int frag_off = fragment_offset(lane);

  int n_tiles = a.n_tiles, tiles_m = g.tiles_m;
  if (GROUPED) {
    tiles_m = 0;
    for (int e = 0, begin = 0; e < a.n_groups; ++e) {
      const int end = segment_end(a, e, begin);
      tiles_m += (end - begin + kTileRows - 1) / kTileRows;
      begin = end;
    }
    n_tiles = tiles_m * g.tiles_n;
    if (kCuts) {
      // The tiles past the last whole round of the grid: rounds of work items, each as long as its K-blocks plus
      // about 8 for the start of a tile and the exchange (uniform: every block arrives at the same shift).
      const int grid = (int)gridDim.x;
      const int full = n_tiles / grid * grid, rest = n_tiles - full;
      int best = 0, best_cost = g.KB;
      for (int sh = 1; sh <= a.cut_shift; ++sh) {
        if ((rest << sh) * JN > kMaxCutItems) break;  // slots for the partial sums
        const int cost = ((rest << sh) + grid - 1) / grid * ((g.KB >> sh) + 8);
        if (cost < best_cost) { best_cost = cost; best = sh; }
      }
      a.cut_shift = best;
      a.cut_steps = g.KB >> best;
      a.cut_full = best != 0 ? full : n_tiles;
    }
  }
  // steps of this block: whole tiles blockIdx.x, blockIdx.x + gridDim.x, ... or one contiguous range
  int pos = (int)blockIdx.x, first_idx = (int)blockIdx.x, first_kb = 0, total;
  if (SK) {
    // ranges that are neighbours in the step order go to one XCD (block ids congruent mod 8)
    if (a.sk_split) {
      // position of this block in XCD-major order (block b runs on XCD b mod 8), then (cut, tile) in that order
      const int x = (int)(blockIdx.x & 7), per = (int)(gridDim.x >> 3), extra = (int)(gridDim.x & 7);
      const int idx = x * per + (x < extra ? x : extra) + (int)(blockIdx.x >> 3);
      const int cut = idx / a.n_tiles;
      pos = (idx - cut * a.n_tiles) * a.sk_split + cut;
    } else if ((gridDim.x & 7) == 0) {
      pos = (int)(blockIdx.x & 7) * (int)(gridDim.x >> 3) + (int)(blockIdx.x >> 3);
    }
    const int s0 = sk_range_begin(a, pos);
    total = a.sk_q + (pos < a.sk_r ? 1 : 0);
    first_idx = s0 / g.KB;
    first_kb = s0 - first_idx * g.KB;
  } else {
    // (a grouped launch sizes its grid for an upper bound of the tile count: the blocks past the real one leave)
    if (kCuts && a.cut_shift != 0) {
      const int cut_items = (n_tiles - a.cut_full) << a.cut_shift;
      const int mine = (cut_items - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
      total = a.cut_full / (int)gridDim.x * g.KB + (mine > 0 ? mine * a.cut_steps : 0);
    } else {
      const int my_tiles = (n_tiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
      total = my_tiles > 0 ? my_tiles * g.KB : 0;
    }
  }
  if (total <= 0) return;  // uniform over the block
  for (int i = (int)(blockIdx.x & 15) * a.stagger; i > 0; --i) __builtin_amdgcn_s_sleep(15);

  // ---- the stage being loaded
  Walk lw;
  lw.start(a, first_idx, first_kb, n_tiles, tiles_m);
  LoadShare share = {};
  auto set_load_tile = [&]() __attribute__((always_inline)) {
    if (GROUPED && a.gather_index != nullptr && wave < 4) {
      const int valid = lw.m_end - lw.m0;
      share.set_gathered(g, a.gather_index, a.index_div, a.x_rows, lw.m0, valid < kTileRows ? valid : kTileRows, lane, wave);
    } else {
      share.template set_tile<kTileRows>(g, lw.m0, lw.n0, wave, lane, lw.m_end, GROUPED ? (int64_t)lw.group * a.w_group_stride : 0);
    }
  };
  set_load_tile();
  share.ptr += (int64_t)(kCuts ? lw.kb : first_kb) * 128;
  int loaded = 0, w_slot = 0, x_slot = 0;  // stages issued by this wavefront; LDS slots of the next stage
  // (short tiles: the activation rows past the tile's 64 JN are never read, and group A leaves their loads out)
  constexpr int kXLoadsPerWave = JN < kTM ? 2 * JN : kSlabsPerWave;
  auto issue_stage_part = [&](int q) __attribute__((always_inline)) {
    if (JN < kTM && grp == 0 && q >= kXLoadsPerWave) return;
    const uint32_t region = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    const uint32_t stage = grp ? (uint32_t)(w_slot * kWStageBytes) : (uint32_t)(kXReg + x_slot * kXStBytes);
    share.issue_one(region + stage + (uint32_t)(wave & 3) * 1024u, q);
  };
  auto finish_stage = [&]() __attribute__((always_inline)) {
    ++loaded;
    w_slot = (w_slot + 1 == kWSt) ? 0 : w_slot + 1;
    x_slot ^= 1;
    if (__builtin_expect(lw.next(a), 0)) {
      if (lw.inside(a)) {
        if (ALIGNED) share.set_ptr(g, lw.m0, lw.n0, wave);
        else set_load_tile();
        if (kCuts) share.ptr += (int64_t)lw.kb * 128;
      }
    } else {
      share.ptr += 128;
    }
  };
  auto issue_stage_all = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < kSlabsPerWave; ++q) issue_stage_part(q);
    finish_stage();
  };

  // ---- the step whose activation scales are being fetched: four rows per lane, 32-bit byte offsets from
  // a uniform pointer that moves along K (the host checks that M * row stride fits)
  Walk sw;
  sw.start(a, first_idx, first_kb, n_tiles, tiles_m);
  uint32_t xs_off[kTM] = {0u, 0u, 0u, 0u};
  const float* xs_ptr = g.xs;
  // offsets are relative to the tile's first row; rows past the edge read the last row's scale
  const bool gathered = GROUPED && a.gather_index != nullptr;  // uniform
  auto set_scale_offsets = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < kTM; ++j) {
      int r = wm0 + j * 16 + l16;
      const int last = sw.m_end - 1 - sw.m0;
      r = r < last ? r : last;
      if (gathered) {  // the scales of the source row, relative to the first row of the scale matrix
        int src = a.gather_index[sw.m0 + r] / a.index_div;
        r = src < 0 ? 0 : (src < a.x_rows ? src : a.x_rows - 1);
      }
      xs_off[j] = (uint32_t)r * (uint32_t)g.xs_rs * 4u;
    }
  };
  auto set_scale_tile = [&]() __attribute__((always_inline)) {
    if (!ALIGNED) set_scale_offsets();
    xs_ptr = gathered ? g.xs : g.xs + (int64_t)sw.m0 * g.xs_rs;
    if (kCuts) xs_ptr += (int64_t)sw.kb * g.xs_cs;
  };
  if (MODE == kModeBlock) {
    set_scale_offsets();
    set_scale_tile();
    if (!kCuts) xs_ptr += (int64_t)first_kb * g.xs_cs;
  }
  auto advance_scales = [&]() __attribute__((always_inline)) {
    if (__builtin_expect(sw.next(a), 0)) set_scale_tile(); else xs_ptr += g.xs_cs;
  };
  float xs_nxt[kTM] = {0.f, 0.f, 0.f, 0.f};
  auto request_scales = [&]() __attribute__((always_inline)) {
    if (MODE != kModeBlock) return;
    const float* const base = uniform_ptr(xs_ptr);
#pragma unroll
    for (int j = 0; j < kTM; ++j) load_f32_untracked(xs_nxt[j], xs_off[j], base);
  };

  // ---- the step being multiplied; its weight-block scale is one scalar load per step
  Walk cw;
  cw.start(a, first_idx, first_kb, n_tiles, tiles_m);
  const int nb_last = (g.N - 1) >> 7;
  auto ws_row = [&]() __attribute__((always_inline)) -> const float* {
    int nb = (cw.n0 + wn0) >> 7;
    nb = nb < nb_last ? nb : nb_last;
    return g.ws + (GROUPED ? (int64_t)cw.group * a.ws_group_stride : 0) + (int64_t)nb * g.ws_rs + (kCuts ? (int64_t)cw.kb * g.ws_cs : 0);
  };
  const float* ws_ptr = MODE == kModeBlock ? ws_row() + (kCuts ? 0 : (int64_t)first_kb * g.ws_cs) : nullptr;

  // ---- prologue: A has stage 0 in flight, B stages 0 and 1; scales of step 0
  issue_stage_all();
  if (grp == 1 && total > 1) issue_stage_all();
  if (kWSt > kWStages && grp == 1 && total > 2) issue_stage_all();
  request_scales();
  if (MODE == kModeBlock && total > 1) advance_scales();  // fetch(T) asks for the scales of step T+1
  wait_vmem_all();
  __builtin_amdgcn_s_barrier();
  if (grp == 1) __builtin_amdgcn_s_barrier();  // B runs one slot behind A
  __builtin_amdgcn_s_setprio(kFetchPrio);

  v4f acc[kTN][JN];
#pragma unroll
  for (int t = 0; t < kTN; ++t)
#pragma unroll
    for (int j = 0; j < JN; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};

  // A finished tile is stored at the end of its wavefront's next fetch slot, under the partner's MFMAs.
  // A tile of which this block computed only some K-blocks (stream-K) goes through finish_partial_tile at
  // the start of that slot instead: its waits may stall the pair for a few microseconds, twice per block.
  bool pending = false;
  int pend_m = 0, pend_n = 0, pend_idx = 0, pend_m_end = 0;
  auto clear_acc = [&]() __attribute__((always_inline)) {
    // (a second copy of the multiply phase that overwrites instead of accumulating makes the register
    // allocator shuffle the accumulators through scratch at the join; zeroing costs 128 moves per tile)
#pragma unroll
    for (int t = 0; t < kTN; ++t)
#pragma unroll
      for (int j = 0; j < JN; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};
    pending = false;
  };
  auto flush_whole_tile = [&]() __attribute__((always_inline)) {
    if constexpr (kCutsInLoop) {
      if (pend_idx >= a.cut_full) {
        wait_vmem<0>();
        finish_cut_tile<GROUPED, JN, F16>(a, acc, pend_idx - a.cut_full, pend_m, pend_n, pend_m_end, wave, lane, l16, lg);
        clear_acc();
        return;
      }
    }
    store_tile<MODE, ALIGNED, GROUPED, JN, F16>(g, acc, pend_m, pend_n, l16, lg, pend_m_end, GROUPED && a.c_rows > 0 ? a.row_index : nullptr,
                                                a.c_rows, a.row_weight);
    clear_acc();
  };
  auto flush_partial_tile = [&]() __attribute__((always_inline)) {
    wait_vmem<0>();
    if constexpr (SK) finish_partial_tile<MODE, F16>(a, acc, pend_idx, pos, pend_m, pend_n, wave, lane, l16, lg);
    clear_acc();
  };

  int rw_slot = 0, rx_slot = 0;  // LDS slots of the stage being read
  // The stores of a finished tile are counted by vmcnt like the loads, in issue order.  Where their number is
  // known (kStoresPerTile, aligned shapes in block mode) the waits of the following slots allow that many
  // younger operations more, so that nobody waits for the stores to reach memory before the first load issued
  // after them is needed: all compute units finish tiles at about the same time, and 32 MB of results take
  // several microseconds to drain.
  constexpr bool kRelaxedStoreWaits = ALIGNED && MODE == kModeBlock;
  bool flushed_prev = false;  // this wavefront stored a tile in its previous fetch phase
  auto run_steps = [&](int t_begin, int t_end) __attribute__((always_inline)) {
  flushed_prev = false;  // every instance of this loop ends with all vector-memory operations complete
  for (int T = t_begin; T < t_end; ++T) {
    // ================= fetch(T)
    // Scales of this step were requested a step ago; the only younger vector-memory operations are the eight
    // tile loads that followed them (for A those have landed as well: it waited at the end of its multiply).
    float xs[kTM], sc[kTM];
    int se[kTM], swe = 0;  // POW2: exponents of the activation-row scales and of the weight-block scale
    const bool more = T + 1 < total;
    float ws = 1.f;
    if (MODE == kModeBlock) {
      if (kRelaxedStoreWaits && flushed_prev) wait_and_take<8 + kStoresPerTile>(xs, xs_nxt);
      else if (JN < kTM && grp == 0) wait_and_take<kXLoadsPerWave>(xs, xs_nxt);
      else wait_and_take<8>(xs, xs_nxt);
      if (more) request_scales();  // of step T+1; the pointer was moved there a step ago
      ws = *(const __attribute__((address_space(4))) float*)ws_ptr;
    }
    const uint8_t* const tw = lds + rw_slot * kWStageBytes + (wn0 >> 4) * 2048;
    const uint8_t* const tx = lds + kXReg + rx_slot * kXStBytes + (wm0 >> 4) * 2048;
    // All activation fragments and the first two weight fragments (the other six follow during the multiply,
    // each two MFMA rows before its use), interleaved with this wavefront's eight tile loads: the address
    // unit takes ~45 cycles per 1 KB load and the LDS ~25 per fragment half, and a wavefront that issues
    // either kind back to back waits for the unit each time.
    //   A loads the activations of stage T+1 into the slot that fetch(T-1) read,
    //   B the weights of stage T+2 into the slot that multiply(T-1) left a slot ago.
    // Past the last stage the loads are repeated from the last address into a slot nobody reads any more:
    // cheaper than a branch per load, and the wait counts below stay the same on every step.
    v8i xf[JN], wr[3];
    v4f p_tail[2];  // results of the step's last two MFMAs, scaled into the sums after the barrier that ends the slot
    (void)p_tail;
    issue_stage_part(0);
    xf[0] = read_frag(tx, 0, frag_off);
    issue_stage_part(1);
    if (JN > 1) xf[1 % JN] = read_frag(tx, 1, frag_off);
    issue_stage_part(2);
    if (JN > 2) xf[2 % JN] = read_frag(tx, 2, frag_off);
    issue_stage_part(3);
    if (JN > 3) xf[3 % JN] = read_frag(tx, 3, frag_off);
    issue_stage_part(4);
    wr[0] = read_frag(tw, 0, frag_off);
    issue_stage_part(5);
    wr[1] = read_frag(tw, 1, frag_off);
    issue_stage_part(6);
    issue_stage_part(7);
    // scalar bookkeeping of the next step, under the latency of the LDS reads (in the multiply phase every
    // extra instruction delays the MFMAs: a wavefront issues one instruction in ~6 cycles, and the MFMA with
    // its four FMAs fills the 32 cycles the matrix pipe takes)
    if (loaded < total) finish_stage();
    if (MODE == kModeBlock && T + 2 < total) advance_scales();
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): fragments are in registers
    // B's weights of stage T+1, issued a step ago, must have landed before the barrier; the scale requests
    // and the tile loads of this slot are younger.
    if (grp == 1) {
      if (kRelaxedStoreWaits && flushed_prev) {
        if (more) wait_vmem<12 + kStoresPerTile>(); else wait_vmem<8 + kStoresPerTile>();
      } else if (kWSt > kWStages) {
        // (one more stage is younger; the in-order wait for the scales at the start of the slot has covered stage T+1)
        if (more && MODE == kModeBlock) wait_vmem<20>(); else wait_vmem<16>();
      } else {
        if (more && MODE == kModeBlock) wait_vmem<12>(); else wait_vmem<8>();
      }
    }
    if (MODE == kModeBlock) {
      if (POW2) {
        swe = e8m0_of(ws);
#pragma unroll
        for (int j = 0; j < JN; ++j) se[j] = e8m0_of(xs[j]);
      } else {
#pragma unroll
        for (int j = 0; j < JN; ++j) sc[j] = xs[j] * ws;
      }
    }
    const bool flushed_now = pending;
    if (pending) flush_whole_tile();  // after the waits, so that no wait of this slot covers the stores
    __builtin_amdgcn_s_barrier();

    // ================= multiply(T)
    __builtin_amdgcn_s_setprio(kMultiplyPrio);
    if (MODE >= kModeRowColI8) {
      // int8, bf16, fp16: per row of tiles first the JN products of the lower K half, then those of the upper
#pragma unroll
      for (int t = 0; t < kTN; ++t) {
#pragma unroll
        for (int j = 0; j < JN; ++j) {
          mfma_accumulate_half<MODE>(acc[t][j], wr[t % 3], xf[j], 0);
          if (j == 0 && t + 2 < kTN) wr[(t + 2) % 3] = read_frag(tw, t + 2, frag_off);
        }
#pragma unroll
        for (int j = 0; j < JN; ++j) mfma_accumulate_half<MODE>(acc[t][j], wr[t % 3], xf[j], 1);
      }
    } else if (MODE != kModeBlock) {
      // row/column mode: the matrix pipe accumulates; scales and bias wait for the epilogue
#pragma unroll
      for (int st = 0; st < kTN * JN; ++st) {
        const int t = st / JN, j = st % JN;
        mfma_accumulate(acc[t][j], wr[t % 3], xf[j]);
        if (j == 0 && t + 2 < kTN) wr[(t + 2) % 3] = read_frag(tw, t + 2, frag_off);
      }
    } else if (POW2) {
#pragma unroll
      for (int st = 0; st < kTN * JN; ++st) {
        const int t = st / JN, j = st % JN;
        mfma_scaled_accumulate(acc[t][j], wr[t % 3], xf[j], swe, se[j]);
        if (j == 0 && t + 2 < kTN) wr[(t + 2) % 3] = read_frag(tw, t + 2, frag_off);
      }
    } else {
      v4f p[3];
#pragma unroll
      for (int st = 0; st < kTN * JN; ++st) {
        const int t = st / JN, j = st % JN;
        p[st % 3] = mfma_partial(wr[t % 3], xf[j]);
        // refill the ring after the row's first MFMA: the wait the compiler puts before that MFMA then
        // covers only reads issued a whole row earlier
        if (j == 0 && t + 2 < kTN) wr[(t + 2) % 3] = read_frag(tw, t + 2, frag_off);
        if (st >= 2) scale_into<0>(acc[(st - 2) / JN][(st - 2) % JN], p[(st - 2) % 3], sc[(st - 2) % JN]);
      }
      // The FMAs of the last two MFMAs wait until after the barrier below: they need the matrix pipe's last
      // results (44 cycles after the last MFMA's issue), and while this wavefront waited for them before the barrier,
      // the partner, whose MFMAs were ready, waited too.  (Short tiles keep them here: their steps are set by the
      // weight stream, and with the FMAs behind the barrier a step of 64-row tiles took a quarter longer.)
      if (kDeferTail) {
        p_tail[0] = p[(kTN * JN - 2) % 3]; p_tail[1] = p[(kTN * JN - 1) % 3];
      } else {
        constexpr int L = kTN * JN;
        scale_into<0>(acc[(L - 2) / JN][(L - 2) % JN], p[(L - 2) % 3], sc[(L - 2) % JN]);
        scale_into<4>(acc[(L - 1) / JN][(L - 1) % JN], p[(L - 1) % 3], sc[(L - 1) % JN]);
      }
    }
    __builtin_amdgcn_s_setprio(kFetchPrio);
    if (grp == 0) {  // A's share of stage T+1 has landed
      if (kRelaxedStoreWaits && flushed_now) wait_vmem<kStoresPerTile>(); else wait_vmem_all();
    }
    flushed_prev = flushed_now;
    __builtin_amdgcn_s_barrier();
    if (MODE == kModeBlock && !POW2 && kDeferTail) {
      // (wait states between the last MFMA and the FMA that reads it: the four FMAs issued behind that MFMA, the
      // priority change, the barrier, two here, four FMAs, two more)
      constexpr int L = kTN * JN;
      scale_into<2>(acc[(L - 2) / JN][(L - 2) % JN], p_tail[0], sc[(L - 2) % JN]);
      scale_into<2>(acc[(L - 1) / JN][(L - 1) % JN], p_tail[1], sc[(L - 1) % JN]);
    }

    // ================= next step; a finished tile is stored in this wavefront's next fetch slot
    rw_slot = (rw_slot + 1 == kWSt) ? 0 : rw_slot + 1;
    rx_slot ^= 1;
    pend_m = cw.m0 + wm0; pend_n = cw.n0 + wn0; pend_idx = cw.idx; pend_m_end = cw.m_end;
    pending = __builtin_expect(cw.next(a), 0);
    if (MODE == kModeBlock) {
      if (pending) ws_ptr = ws_row(); else ws_ptr += g.ws_cs;
    }
  }
  // The scales requested for the next step are on their way into registers the compiler knows nothing about,
  // and it copies them where one instance of this loop hands over to the next (three with stream-K): they must
  // have arrived before that.  The operands make the copies come after the wait.
  if (MODE == kModeBlock) {
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(xs_nxt[0]), "+v"(xs_nxt[1]), "+v"(xs_nxt[2]), "+v"(xs_nxt[3]) : : "memory");
  }
  };

  if (SK) {
    // A range is [part of a tile] [whole tiles] [part of a tile]; the hot loop runs once for each piece and
    // the partial pieces are finished between the runs, outside any loop.
    const int n_head = first_kb != 0 ? (total < g.KB - first_kb ? total : g.KB - first_kb) : 0;
    const int n_whole = (total - n_head) / g.KB * g.KB;
    if (n_head > 0) {
      run_steps(0, n_head);
      flush_partial_tile();
    }
    run_steps(n_head, n_head + n_whole);
    if (n_head + n_whole < total) {
      run_steps(n_head + n_whole, total);  // (stores the last whole tile in its first fetch slot)
      flush_partial_tile();
    } else if (pending) {
      flush_whole_tile();
    }
  } else if (kCuts && !kCutsInLoop) {
    const int n_whole = a.cut_shift != 0 ? a.cut_full / (int)gridDim.x * g.KB : total;
    run_steps(0, n_whole);
    if (pending) flush_whole_tile();
    for (int t0 = n_whole; t0 < total; t0 += a.cut_steps) {  // this block's work items of cut tiles
      run_steps(t0, t0 + a.cut_steps);
      wait_vmem<0>();
      finish_cut_tile<GROUPED, JN, F16>(a, acc, pend_idx - a.cut_full, pend_m, pend_n, pend_m_end, wave, lane, l16, lg);
      clear_acc();
    }
  } else {
    run_steps(0, total);
    if (pending) flush_whole_tile();
  }
  wait_vmem_all();  // the tile loads repeated past the last stage
  if (grp == 0) __builtin_amdgcn_s_barrier();  // pairs with B's extra barrier at the start
}

// Stream-K pays when whole-tile rounds leave compute units idle: `steps` K-blocks per block either way.
struct SkPlan {
  bool use;
  int grid, q, r;
  int split;  // != 0: tiles cut into `split` equal ranges each (grid = tiles * split), see PpArgs::sk_split
};
SkPlan plan_stream_k(int64_t tiles, int KB, int cus) {
  SkPlan p = {false, 0, 0, 0, 0};
  const int64_t total = tiles * KB;
  if (cus < 8 || total < cus || total > 0x7FFFFFFF) return p;
  const int64_t dp_grid = tiles < cus ? tiles : cus;
  const int64_t dp_steps = ceil_div(tiles, dp_grid) * KB;
  const int64_t q = total / cus;
  // Equal cuts of every tile (PpArgs::sk_split) keep the operand sharing of whole-tile launches, which contiguous
  // ranges of total / cus steps lose unless they happen to cut every tile alike.  They pay when the cuts are long
  // and nearly fill the GPU: measured M = 512, N = 7168, K = 16384 (56 tiles): 4 cuts of 32 steps on 224 units
  // 86 us against 110 us for 256 ranges of 28 steps; M = 1024, same N and K: 2 cuts of 64 steps 125 us against
  // 174 us.  Cuts down to 16 steps on at least half of the units still win (M = 2048, N = 3072, K = 8192, 96 tiles in
  // 2 cuts of 32: 84 -> 70 us; M = 4096, N = 1536, K = 7168, 96 tiles in 2 cuts of 28: 76 -> 65 us; M = 3072,
  // N = 2112, K = 7168: 85 -> 73 us); cuts of 8 steps lose to the contiguous ranges.
  const bool ranges_cut_tiles_alike = total % cus == 0 && q > 0 && KB % q == 0;
  if (!ranges_cut_tiles_alike) {
    for (int64_t S = cus / tiles; S >= 2; --S) {
      if (KB % S != 0) continue;
      const int64_t cut = KB / S;
      if (cut < 16 || tiles * S * 2 < (int64_t)cus) break;  // shorter cuts or emptier grids only get worse
      if ((cut + 16) >= dp_steps) break;                         // ~16 steps to publish and add the partial tiles
      p.use = true; p.grid = (int)(tiles * S); p.q = (int)cut; p.r = 0; p.split = (int)S;
      return p;
    }
  }
  // Measured on DeepSeek-V3 shapes, M = 128 ... 4096, in units of a whole-tile K-block: ranges that start at
  // different K offsets stop sharing operand panels in their XCD's L2, which makes a K-block about 1.35 times as
  // expensive, and the tiles are finished only after the slowest of their ranges, which adds about 14 K-blocks
  // plus 0.3 of a tile's K loop.  Stream-K is chosen when it still comes out ahead, and never with more than 16
  // ranges a tile.
  if (q * 16 < KB) return p;
  const int64_t sk_steps_x10 = (ceil_div(total, cus) * 27 + 1) / 2 + 3 * KB + 140;
  if (sk_steps_x10 >= dp_steps * 10) return p;
  p.use = true;
  p.grid = cus;
  p.q = (int)q;
  p.r = (int)(total % cus);
  return p;
}

// Whole rounds plus a few tiles: the last round would keep tiles % cus units busy for a whole K loop.  Those tiles
// go to a second launch instead, every one cut into `split` equal ranges (PpArgs::sk_split, tile_base) so that
// more units share them.  What limits it is the exchange of partial tiles (256 KB each way per block, through
// memory): measured ~0.25 K-block times per block of the second launch, so it gets at most 128 blocks and is taken
// only when the sum still comes out 5 % ahead.  M = 4096, N = 4608, K = 7168 (288 tiles on 256 units, 32 x 4
// ranges of 14): 169 -> 149 us; M = 2304, N = 8192, K = 8192: 192 -> 168 us; with 8 ranges of 7 (256 blocks) the
// first shape takes 176 us.
struct TailPlan {
  bool use;
  int full, tail, split, cut, grid;
};
TailPlan plan_tail(int64_t tiles, int KB, int cus) {
  TailPlan p = {false, 0, 0, 0, 0, 0};
  if (cus < 8 || tiles <= cus || tiles > 0x3FFFFFFF) return p;
  const int64_t tail = tiles % cus;
  if (tail == 0 || tail * 4 > cus) return p;
  int64_t S = (cus / 2) / tail;
  if (S > 16) S = 16;
  while (S >= 2 && KB % S != 0) --S;
  if (S < 2 || KB / S < 4) return p;
  const int64_t rounds = ceil_div(tiles, (int64_t)cus);
  const int64_t now = rounds * KB, then = (rounds - 1) * KB + KB / S + tail * S / 4;
  if (then * 100 > now * 95) return p;
  p.use = true;
  p.full = (int)(tiles - tail); p.tail = (int)tail; p.split = (int)S; p.cut = (int)(KB / S); p.grid = (int)(tail * S);
  return p;
}

// Activation scales [M, K/128] -> [K/128, M].  The GEMM reads four scales per lane and K-block, for rows 16
// apart; with K-major rows that is a separate 128-byte line from L2 for every row and K-block (the tile loads
// keep sweeping the L1), as many line requests as the tiles themselves need, and the tile loads queue behind
// them in the address unit: measured 20 % of the run time on K = 16384.  From the transposed copy a
// wavefront's 64 scales of a K-block are 256 contiguous bytes.
// One thread per row and 4 K-blocks: reads run along a row (16-byte loads where the layout allows), writes
// run along M and are contiguous over the threads of a block.
constexpr int kTransposeKbPerBlock = 4;  // (16: a quarter of the blocks and 3 us instead of 2 on [4096, 56])
__global__ __launch_bounds__(256) void transpose_scales_kernel(const float* __restrict__ xs, int64_t rs, int64_t cs, int M,
                                                               int KB, float* __restrict__ out) {
  const int m = (int)blockIdx.x * 256 + (int)threadIdx.x;
  const int kb0 = (int)blockIdx.y * kTransposeKbPerBlock;
  if (m >= M) return;
  const float* const row = xs + (int64_t)m * rs;
  const bool vec = cs == 1 && (rs & 3) == 0 && ((uintptr_t)xs & 15) == 0;
#pragma unroll
  for (int i = 0; i < kTransposeKbPerBlock; i += 4) {
    const int kb = kb0 + i;
    float v[4];
    if (vec && kb + 4 <= KB) {
      const v4f q = *reinterpret_cast<const v4f*>(row + kb);
      v[0] = q[0]; v[1] = q[1]; v[2] = q[2]; v[3] = q[3];
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = kb + e < KB ? row[(int64_t)(kb + e) * cs] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (kb + e < KB) out[(int64_t)(kb + e) * M + m] = v[e];
  }
}

// The extra launch costs ~5 us (it is all latency) and saves ~10 % of the GEMM: worth it for rows of scales at
// least this many floats apart and a GEMM of more than ~50 us (a K-block takes ~1.66 us per round of tiles).
constexpr int64_t kTransposeMinRowStride = 8;
bool transposition_pays(int64_t tiles, int64_t KB, int cus) {
  if (KB < kTransposeMinRowStride) return false;
  const SkPlan sk = plan_stream_k(tiles, (int)KB, cus);
  const double steps = sk.use ? 1.35 * (sk.q + 1) + 0.3 * KB + 14 : (double)ceil_div(tiles, (int64_t)cus) * (double)KB;
  return steps * 1.66 > 50.0;
}
size_t transposed_scales_bytes(int64_t M, int64_t KB) { return (size_t)((M * KB * 4 + 255) / 256 * 256); }

// Short tiles of grouped problems (the JN = 1 instantiation) and their cuts along K.
constexpr int kShortTileRows = 64;
constexpr size_t kCutSlotBytes = (size_t)8 * kTN * 256 * 4;  // a work item's partial sums: 8 wavefronts x 16 x 128 floats
// Largest number of cuts per tile of the last round, as a shift (the kernel picks among 0..this from the real tile
// count): whole K-blocks, at least 8 per cut, and slots for a round short of one tile.
// (256-row tiles, jn = 4: a round short of one tile would need four times the slots; the kernel, which knows how many
// tiles the last round really holds, takes a shift only while their work items fit)
int max_cut_shift(int grid, int KB, int jn) {
  int sh = 0;
  while (sh < 2 && KB % (2 << sh) == 0 && (KB >> (sh + 1)) >= 8 && (jn == kTM || ((int64_t)(grid - 1) << (sh + 1)) * jn <= kMaxCutItems)) ++sh;
  return sh;
}

// The instantiation that serves a launch.
struct KernelChoice {
  bool grouped;
  int short_jn;  // grouped problems on short tiles: 16-row fragments per wavefront (1 or 2), else 0
  int mode;
  bool sk, aligned, pow2;
};
template <bool F16>
void (*pick_kernel(const KernelChoice& c))(PpArgs) {
  if (c.grouped)
    return c.short_jn == 1   ? fp8_gemm_pingpong_kernel<false, kModeBlock, false, true, false, 1, F16>
           : c.short_jn == 2 ? fp8_gemm_pingpong_kernel<false, kModeBlock, false, true, false, 2, F16>
                             : fp8_gemm_pingpong_kernel<false, kModeBlock, false, true, false, kTM, F16>;
  if (c.mode == kModeRowColI8) {
    if (c.sk)
      return c.aligned ? fp8_gemm_pingpong_kernel<true, kModeRowColI8, true, false, false, kTM, F16>
                       : fp8_gemm_pingpong_kernel<true, kModeRowColI8, false, false, false, kTM, F16>;
    return c.aligned ? fp8_gemm_pingpong_kernel<false, kModeRowColI8, true, false, false, kTM, F16>
                     : fp8_gemm_pingpong_kernel<false, kModeRowColI8, false, false, false, kTM, F16>;
  }
  // (16-bit operands: their entry point has no workspace, so tiles are never shared)
  if (c.mode == kModeRowColBF16)
    return c.aligned ? fp8_gemm_pingpong_kernel<false, kModeRowColBF16, true, false, false, kTM, F16>
                     : fp8_gemm_pingpong_kernel<false, kModeRowColBF16, false, false, false, kTM, F16>;
  if (c.mode == kModeRowColF16)
    return c.aligned ? fp8_gemm_pingpong_kernel<false, kModeRowColF16, true, false, false, kTM, F16>
                     : fp8_gemm_pingpong_kernel<false, kModeRowColF16, false, false, false, kTM, F16>;
  if (c.mode != kModeBlock) {
    if (c.sk)
      return c.aligned ? fp8_gemm_pingpong_kernel<true, kModeRowCol, true, false, false, kTM, F16>
                       : fp8_gemm_pingpong_kernel<true, kModeRowCol, false, false, false, kTM, F16>;
    return c.aligned ? fp8_gemm_pingpong_kernel<false, kModeRowCol, true, false, false, kTM, F16>
                     : fp8_gemm_pingpong_kernel<false, kModeRowCol, false, false, false, kTM, F16>;
  }
  if (c.pow2) {
    if (c.sk)
      return c.aligned ? fp8_gemm_pingpong_kernel<true, kModeBlock, true, false, true, kTM, F16>
                       : fp8_gemm_pingpong_kernel<true, kModeBlock, false, false, true, kTM, F16>;
    return c.aligned ? fp8_gemm_pingpong_kernel<false, kModeBlock, true, false, true, kTM, F16>
                     : fp8_gemm_pingpong_kernel<false, kModeBlock, false, false, true, kTM, F16>;
  }
  if (c.sk)
    return c.aligned ? fp8_gemm_pingpong_kernel<true, kModeBlock, true, false, false, kTM, F16>
                     : fp8_gemm_pingpong_kernel<true, kModeBlock, false, false, false, kTM, F16>;
  return c.aligned ? fp8_gemm_pingpong_kernel<false, kModeBlock, true, false, false, kTM, F16>
                   : fp8_gemm_pingpong_kernel<false, kModeBlock, false, false, false, kTM, F16>;
}

// Every instantiation uses all of a compute unit's LDS, which a kernel has to be allowed once per device.  The
// kernels are few: a short table of the ones seen so far, under a lock.
int allow_full_lds(void (*kern)(PpArgs)) {
  constexpr int kMaxKernels = 64;
  static std::mutex lock;
  static const void* seen[kMaxKernels];
  static PerDeviceFlags raised[kMaxKernels];
  static int n_seen = 0;
  const void* const k = reinterpret_cast<const void*>(kern);
  std::lock_guard<std::mutex> guard(lock);
  int i = 0;
  while (i < n_seen && seen[i] != k) ++i;
  if (i == n_seen) {
    if (n_seen == kMaxKernels) FG_FAIL(FG_ERR_LAUNCH, "fp8 gemm: kernel table full");
    seen[n_seen++] = k;
  }
  const hipError_t e = raise_dynamic_lds_limit(raised[i], kLdsBytes, k);
  if (e != hipSuccess) FG_FAIL(FG_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", kLdsBytes, hipGetErrorString(e));
  return FG_OK;
}

int launch_block(const GemmArgs& g, int mode, void* workspace, size_t workspace_bytes, hipStream_t stream,
                 const GroupedGemm* grouped = nullptr) {
  PpArgs a = {};
  a.g = g;
  a.g.tiles_m = (int)ceil_div(g.M, kBM);
  // Grouped problems with few rows per segment take tiles of 64 or 128 rows (the JN = 1 and 2 instantiations).  The
  // host sees only the average; a segment longer than a tile reads its weights once per tile, and where the tiles
  // are few (at most half the compute units when every segment has one) a longer segment also costs a round of its
  // own, so those take the next tile height sooner.  Measured on 8 segments, [28672, 4096] | [4096, 14336] weights
  // each (896 | 128 tiles), us for 256- / 64- / 128-row tiles by rows a segment on average:
  //    16: 333 222 249 | 203 112 125     32: 295 223 240 | 207 170 128     64: 303 295 243 | 222 178 192
  //    96: 303 336 288 | 219 181 189    128: 293 415 318 | 202 217 182     256: 404 705 463 | 213 351 269
  int short_jn = 0;
  if (grouped != nullptr) {
    const int64_t E = grouped->n_groups;
    const bool few_tiles = E * ceil_div(g.N, kBN) * 2 <= cu_count();
    if (g.M <= 16 * E) short_jn = 1;
    else if (g.M <= 32 * E) short_jn = few_tiles ? 2 : 1;
    else if (g.M <= 96 * E) short_jn = 2;
    else if (g.M <= 128 * E) short_jn = few_tiles ? 2 : 0;
  }
  const bool short_tiles = short_jn != 0;
  if (grouped != nullptr) {
    // every segment ends with at most one tile that is not full; the kernel counts the real tiles
    const int tile_rows = short_tiles ? kShortTileRows * short_jn : kBM;
    const int64_t bound = g.M / tile_rows + grouped->n_groups;
    a.g.tiles_m = (int)(bound < g.M ? bound : g.M);
    a.groups = grouped->ends; a.n_groups = (int)grouped->n_groups;
    a.w_group_stride = grouped->w_group_stride; a.ws_group_stride = grouped->ws_group_stride;
    a.row_index = grouped->row_index; a.index_div = (int)grouped->index_div; a.x_rows = (int)grouped->x_rows;
    a.gather_index = grouped->index_div > 0 ? grouped->row_index : nullptr;
    a.c_rows = (int)grouped->c_rows; a.row_weight = grouped->row_weight;
  }
  a.g.tiles_n = (int)ceil_div(g.N, kBN);
  const int64_t tiles = (int64_t)a.g.tiles_m * a.g.tiles_n;
  if (tiles > 0x3FFFFFFF) FG_FAIL(FG_ERR_UNSUPPORTED, "fp8 gemm: too many tiles");
  a.n_tiles = (int)tiles;
  {
    const uint64_t d = 4ull * (uint64_t)a.g.tiles_n;
    // n * magic >> 40 == n / d for every n with n * d < 2^40 (the tile numbers of whole problems are below `tiles`)
    a.group4_magic = (d > 0 && (uint64_t)tiles * d < (1ull << 40)) ? ((1ull << 40) + d - 1) / d : 0;
  }
  const int cus = cu_count();
  int grid = tiles < cus ? (int)tiles : cus;
  // Stream-K is an optimisation the workspace enables: without one (or with a small one) whole tiles go round-robin.
  SkPlan sk = plan_stream_k(tiles, g.KB, cus);
  if (grouped != nullptr) sk.use = false;  // ranges of steps would need the tile count on the host
  TailPlan tp = plan_tail(tiles, g.KB, cus);
  if (sk.use || grouped != nullptr || mode != kModeBlock) tp.use = false;
  size_t sk_bytes = sk.use ? (size_t)sk.grid * 2 * kPartialSlotBytes : (tp.use ? (size_t)tp.grid * 2 * kPartialSlotBytes : 0);
  a.cut_steps = g.KB;
  if (grouped != nullptr) {
    // (the grid is the compute units, also where the bound of the tile count is lower: cuts may fill them)
    const int sh = max_cut_shift(cus, g.KB, short_tiles ? short_jn : kTM);
    const size_t bytes = (size_t)kMaxCutItems * kCutSlotBytes;
    if (sh > 0 && workspace != nullptr && (uintptr_t)workspace % 16 == 0 && workspace_bytes >= FG_WORKSPACE_COUNTER_BYTES + bytes &&
        (size_t)cus * 8 * 4 <= FG_WORKSPACE_COUNTER_BYTES) {
      a.cut_shift = sh;
      a.counters = reinterpret_cast<unsigned int*>(workspace);
      a.partials = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(workspace) + FG_WORKSPACE_COUNTER_BYTES);
      sk_bytes = bytes;
      grid = (tiles << sh) < cus ? (int)(tiles << sh) : cus;
    }
  }
  const size_t need = FG_WORKSPACE_COUNTER_BYTES + sk_bytes;
  // rows of the activation-scale matrix: the rows of X, which a gathered problem reads through its index
  const int64_t scale_rows = (grouped != nullptr && grouped->row_index != nullptr && grouped->index_div > 0) ? grouped->x_rows : (int64_t)g.M;
  // workspace: [counters][partial tiles, if the shape is one that shares tiles][transposed activation scales]
  // (a grouped problem's tile count is an upper bound that a few hundred rows spread over many segments inflate:
  // there the gathers are few and the transposition, ~5 us whatever the size, does not pay)
  if (mode == kModeBlock && g.xs_rs >= kTransposeMinRowStride && transposition_pays(tiles, g.KB, cus) && workspace != nullptr &&
      (grouped == nullptr || g.M >= 1024) &&
      (uintptr_t)workspace % 16 == 0 &&
      workspace_bytes >= need + transposed_scales_bytes(scale_rows, g.KB)) {
    float* const xs_t = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(workspace) + need);
    FG_LAUNCH(transpose_scales_kernel, dim3((uint32_t)ceil_div(scale_rows, (int64_t)256), (uint32_t)ceil_div(g.KB, kTransposeKbPerBlock)),
                       dim3(256), 0, stream, g.xs, g.xs_rs, g.xs_cs, (int)scale_rows, g.KB, xs_t);
    FG_CHECK_LAUNCH("transpose_scales_kernel");
    a.g.xs = xs_t; a.g.xs_rs = 1; a.g.xs_cs = scale_rows;
  }
  if (sk.use && mode < kModeRowColBF16 && workspace != nullptr && workspace_bytes >= need && (size_t)sk.grid * 8 * 4 <= FG_WORKSPACE_COUNTER_BYTES &&
      (uintptr_t)workspace % 16 == 0) {
    a.sk = 1; a.sk_q = sk.q; a.sk_r = sk.r; a.sk_split = sk.split;
    a.counters = reinterpret_cast<unsigned int*>(workspace);
    a.partials = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(workspace) + FG_WORKSPACE_COUNTER_BYTES);
    grid = sk.grid;
  }
  // Many whole tiles per block, each computed faster than the memory takes a batch of result tiles
  // (256 x 256 bf16 per unit at ~3.3 TB/s; a K-block takes ~1.66 us): the run is bound by the stores, and
  // starting the blocks spread over one tile time lets the stores of some overlap the MFMAs of others
  // (M = 4096, N = 32768, K = 512: 113 -> 98 us).  Everywhere else the delay only costs.
  if (!a.sk && grouped == nullptr && tiles >= 6 * (int64_t)grid) {
    const double tile_us = 1.66 * g.KB, batch_us = grid * 131072.0 / 3.3e6;
    if (tile_us < batch_us) a.stagger = (int)(tile_us * 1.6e3 / 1000.0 / 16 + 0.5);  // 1.6 GHz, ~1000 cycles a sleep, 16 start slots
  }
  const bool aligned = g.M % kBM == 0 && g.N % kBN == 0;
  const bool pow2 = mode == kModeBlock && grouped == nullptr && g.scales_pow2 != 0;
  const bool f16 = g.c_dtype == FG_F16;
  const KernelChoice which = {grouped != nullptr, short_jn, mode, a.sk != 0, aligned, pow2};
  void (*const kern)(PpArgs) = f16 ? pick_kernel<true>(which) : pick_kernel<false>(which);
  if (const int rc = allow_full_lds(kern)) return rc;
  if (tp.use && !a.sk && workspace != nullptr && workspace_bytes >= need && (size_t)tp.grid * 8 * 4 <= FG_WORKSPACE_COUNTER_BYTES &&
      (uintptr_t)workspace % 16 == 0) {
    PpArgs whole = a;
    whole.n_tiles = tp.full;
    whole.stagger = 0;
    FG_LAUNCH(kern, dim3((uint32_t)cus), dim3(kThreads), kLdsBytes, stream, whole);
    FG_CHECK_LAUNCH("fp8_gemm_pingpong_kernel (whole rounds)");
    PpArgs rest = a;
    rest.stagger = 0;
    rest.n_tiles = tp.tail; rest.tile_base = tp.full;
    rest.sk = 1; rest.sk_q = tp.cut; rest.sk_r = 0; rest.sk_split = tp.split;
    rest.counters = reinterpret_cast<unsigned int*>(workspace);
    rest.partials = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(workspace) + FG_WORKSPACE_COUNTER_BYTES);
    KernelChoice tail_choice = which;
    tail_choice.sk = true;
    void (*const shared)(PpArgs) = f16 ? pick_kernel<true>(tail_choice) : pick_kernel<false>(tail_choice);
    if (const int rc = allow_full_lds(shared)) return rc;
    FG_LAUNCH(shared, dim3((uint32_t)tp.grid), dim3(kThreads), kLdsBytes, stream, rest);
    FG_CHECK_LAUNCH("fp8_gemm_pingpong_kernel (last tiles)");
    return FG_OK;
  }
  FG_LAUNCH(kern, dim3((uint32_t)grid), dim3(kThreads), kLdsBytes, stream, a);
  FG_CHECK_LAUNCH("fp8_gemm_pingpong_kernel");
  return FG_OK;
}

}  // namespace

int cu_count() {
  static int cached[kMaxDevices] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

bool pingpong_takes(const GemmArgs& g, int mode, const void* workspace, size_t workspace_bytes) {
  // bf16 rows that take 16-byte stores; activation-scale offsets (bytes from the first row) that fit 32 bits
  if (!(g.M > 64 && (g.c_dtype == FG_BF16 || g.c_dtype == FG_F16) && g.ldc % 8 == 0 && (uintptr_t)g.C % 16 == 0)) return false;
  // 64 < M <= 128 wastes half of every 256-row tile: worth it only where tiles get shared along K (few, deep tiles)
  if (g.M <= 128) {
    const SkPlan sk = plan_stream_k(ceil_div(g.N, kBN), g.KB, cu_count());
    if (!(mode == kModeBlock && sk.use && workspace != nullptr && (uintptr_t)workspace % 16 == 0 &&
          workspace_bytes >= FG_WORKSPACE_COUNTER_BYTES + (size_t)sk.grid * 2 * kPartialSlotBytes))
      return false;
  }
  if (mode != kModeBlock) return true;
  return g.xs_rs >= 0 && g.xs_cs >= 0 && g.ws_rs >= 0 && g.ws_cs >= 0 && (int64_t)g.M * g.xs_rs < (1ll << 29);
}

size_t pingpong_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 64 || K <= 0 || K % 128 != 0) return 0;
  const SkPlan sk = plan_stream_k(ceil_div(M, kBM) * ceil_div(N, kBN), (int)(K / 128), cu_count());
  const int64_t KB = K / 128;
  const TailPlan tp = plan_tail(ceil_div(M, kBM) * ceil_div(N, kBN), (int)(K / 128), cu_count());
  const size_t sk_bytes = sk.use ? (size_t)sk.grid * 2 * kPartialSlotBytes : (tp.use ? (size_t)tp.grid * 2 * kPartialSlotBytes : 0);
  const size_t tr_bytes = transposition_pays(ceil_div(M, kBM) * ceil_div(N, kBN), KB, cu_count())
                              ? transposed_scales_bytes(M, KB) : 0;  // for row-major scales
  return sk_bytes + tr_bytes != 0 ? FG_WORKSPACE_COUNTER_BYTES + sk_bytes + tr_bytes : 0;
}

size_t grouped_workspace_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0 || K % 128 != 0) return 0;
  // (the partial sums of cut short tiles: the number of segments is not known here, the bound of the plan is)
  return FG_WORKSPACE_COUNTER_BYTES + (size_t)kMaxCutItems * kCutSlotBytes + transposed_scales_bytes(M, K / 128);
}

int launch_grouped(const GemmArgs& g, const GroupedGemm& grouped, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  if (!((g.c_dtype == FG_BF16 || g.c_dtype == FG_F16) && g.ldc % 8 == 0 && (uintptr_t)g.C % 16 == 0))
    FG_FAIL(FG_ERR_UNSUPPORTED, "grouped fp8 gemm: the result must be bf16 or fp16 with rows that take 16-byte stores");
  if (!(g.xs_rs >= 0 && g.xs_cs >= 0 && g.ws_rs >= 0 && g.ws_cs >= 0 && (int64_t)g.M * g.xs_rs < (1ll << 29)))
    FG_FAIL(FG_ERR_UNSUPPORTED, "grouped fp8 gemm: scale strides must be non-negative and M * row stride below 2^29");
  if (grouped.n_groups <= 0 || grouped.n_groups > 65536) FG_FAIL(FG_ERR_INVALID_ARG, "grouped fp8 gemm: 1..65536 groups");
  if (grouped.row_index != nullptr && grouped.index_div == 0 && grouped.c_rows == 0)
    FG_FAIL(FG_ERR_INVALID_ARG, "grouped fp8 gemm: index divisor 0 (rows not gathered) leaves row_index without a use unless the results are scattered");
  if (grouped.row_index != nullptr && grouped.index_div != 0) {
    if (grouped.index_div < 1 || grouped.index_div > 0x7FFFFFFF) FG_FAIL(FG_ERR_INVALID_ARG, "grouped fp8 gemm: index divisor %lld", (long long)grouped.index_div);
    if (grouped.x_rows < 1 || grouped.x_rows > 0x7FFFFFFF || grouped.x_rows * g.ldx >= (1ll << 32) || grouped.x_rows * g.xs_rs >= (1ll << 29))
      FG_FAIL(FG_ERR_UNSUPPORTED, "grouped fp8 gemm: %lld gathered rows: the rows of A and of its scales must fit 32-bit byte offsets",
              (long long)grouped.x_rows);
  }
  return launch_block(g, kModeBlock, workspace, workspace_bytes, stream, &grouped);
}

int launch_pingpong(const GemmArgs& g, int mode, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  if (!pingpong_takes(g, mode, workspace, workspace_bytes)) FG_FAIL(FG_ERR_UNSUPPORTED, "fp8 gemm: persistent kernel does not take this problem");
  return launch_block(g, mode, workspace, workspace_bytes, stream);
}

}  // namespace fg

// ---------------------------------------------------------------------------------------------
// Measurement aid: the rate at which the matrix pipes take the multiply phase's instruction stream when nothing
// else happens -- eight wavefronts per compute unit, operands in registers, 32 accumulator tiles per wavefront as in
// the GEMM, no LDS, no memory, no barriers.  with_scale_fmas != 0: every MFMA starts from zero and four FMAs add
// its result times a scale to the accumulators two steps later (the block-scaled form); 0: the MFMAs accumulate
// (the row/column form).  The part holds a lower clock under matrix load than the one its peak is quoted at, and
// how much lower depends on the operand bits: `operands` (at least 64 KB of device memory) supplies them, so a
// benchmark can pass the bytes of its own quantized matrices.  The launch performs
// iterations * 32 * 65536 * 8 * (compute units) flops.
// ---------------------------------------------------------------------------------------------
namespace fg {
namespace {
template <bool SCALE>
__global__ __launch_bounds__(kThreads) void mfma_issue_kernel(const uint8_t* __restrict__ operands, int iterations, float* sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v8i w[3], x[kTM];
  // 7 fragments of 64 lanes x 32 bytes per wavefront, 8 wavefronts: 112 KB would be more than promised; the
  // wavefronts of a block share four fragment sets
  const uint8_t* const base = operands + (size_t)(wave & 3) * 7 * 2048;
#pragma unroll
  for (int i = 0; i < 3; ++i) w[i] = *reinterpret_cast<const v8i*>(base + (size_t)i * 2048 + lane * 32);
#pragma unroll
  for (int j = 0; j < kTM; ++j) x[j] = *reinterpret_cast<const v8i*>(base + (size_t)(3 + j) * 2048 + lane * 32);
  float sc[kTM];
#pragma unroll
  for (int j = 0; j < kTM; ++j) sc[j] = 1.0f + 0.001f * (float)((lane + j) & 15);
  v4f acc[kTN][kTM];
#pragma unroll
  for (int t = 0; t < kTN; ++t)
#pragma unroll
    for (int j = 0; j < kTM; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iterations; ++it) {
    if (SCALE) {
      v4f p[3];
#pragma unroll
      for (int st = 0; st < kTN * kTM; ++st) {
        p[st % 3] = mfma_partial(w[(st / kTM) % 3], x[st % kTM]);
        if (st >= 2) scale_into<0>(acc[(st - 2) / kTM][(st - 2) % kTM], p[(st - 2) % 3], sc[(st - 2) % kTM]);
      }
      constexpr int L = kTN * kTM;
      scale_into<0>(acc[(L - 2) / kTM][(L - 2) % kTM], p[(L - 2) % 3], sc[(L - 2) % kTM]);
      scale_into<4>(acc[(L - 1) / kTM][(L - 1) % kTM], p[(L - 1) % 3], sc[(L - 1) % kTM]);
    } else {
#pragma unroll
      for (int st = 0; st < kTN * kTM; ++st) mfma_accumulate(acc[st / kTM][st % kTM], w[(st / kTM) % 3], x[st % kTM]);
    }
  }
  // the work must not be optimised away; the store happens for no real input
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < kTN; ++t)
#pragma unroll
    for (int j = 0; j < kTM; ++j) sum += acc[t][j][0] + acc[t][j][1] + acc[t][j][2] + acc[t][j][3];
  if (sum == 1.2345678e-30f && sink) sink[0] = sum;
}
}  // namespace
}  // namespace fg

extern "C" int fg_mfma_issue_probe(const void* operands, int iterations, int with_scale_fmas, void* sink, void* stream) {
  using namespace fg;
  if (!operands || (uintptr_t)operands % 32 != 0) FG_FAIL(FG_ERR_INVALID_ARG, "fg_mfma_issue_probe: operands must be a 32-byte aligned device pointer");
  if (iterations < 1) FG_FAIL(FG_ERR_INVALID_ARG, "fg_mfma_issue_probe: %d iterations", iterations);
  const dim3 grid((uint32_t)cu_count()), block(kThreads);
  if (with_scale_fmas) FG_LAUNCH(mfma_issue_kernel<true>, grid, block, 0, (hipStream_t)stream, reinterpret_cast<const uint8_t*>(operands), iterations, reinterpret_cast<float*>(sink));
  else FG_LAUNCH(mfma_issue_kernel<false>, grid, block, 0, (hipStream_t)stream, reinterpret_cast<const uint8_t*>(operands), iterations, reinterpret_cast<float*>(sink));
  FG_CHECK_LAUNCH("mfma_issue_kernel");
  return FG_OK;
}
