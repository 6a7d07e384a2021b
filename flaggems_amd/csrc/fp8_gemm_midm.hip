// FP8 GEMM for 33 <= M <= 64 activation rows on gfx950 (and more rows against small weights, in parts of up to 64): the weight is
// read once, straight from global memory into MFMA operand registers, and the activations come out of LDS.
//
// With up to 64 rows the activation slice of a K-block (64 x 128 bytes) is as large as the 64 weight rows a
// wavefront multiplies it with, so a wavefront that fetches both from global memory moves two bytes for every
// weight byte (the decode kernels do that; they were built for <= 32 rows).  Here a block first copies the
// activation rows of its K range into LDS once (swizzled 16-byte chunks, conflict-free as MFMA fragments) and
// its 4 or 8 wavefronts, each with weight rows of its own, read their fragments from there: no wavefront
// shares an output element with another, so nothing is reduced across wavefronts, and the loop has no barrier.
//
//  * A wavefront owns 16 * RG weight rows (RG = 1, 2, 4) and the K-blocks [split * kb_per_split, ...): per K-block
//    2 * RG 16-byte loads per lane (DEPTH K-blocks in flight, 64 VGPRs), 8 LDS reads, 4 * RG MFMAs.
//  * K is split over gridDim.y blocks only as far as LDS (128 KB of activations: 21 K-blocks of 48 rows, 16 of 64 rows, 8 of
//    128 rows) or the number of wavefronts requires; each wavefront then publishes its sums and the one that arrives last adds the
//    splits' sums in split order (a fixed order: results do not depend on timing) and resets the counter.
//
// Arithmetic as in the other kernels: per K-block products accumulated by the fp8 MFMA, multiplied by
// As[m, kb] * Bs[n / 128, kb] in fp32 (block mode) or accumulated unscaled and scaled at the end (row/column mode).

#include "fp8_gemm_common.h"

namespace fg {
namespace {

// TMX 16-row groups of activations are staged (48, 64 or 128 rows; rows past M repeat the last one and are never
// stored); a block keeps at most 128 KB of them in LDS: 21 K-blocks of 48 rows, 16 of 64, 8 of 128.
constexpr int mid_rows(int tmx) { return 16 * tmx; }
constexpr int mid_stage_bytes(int tmx) { return mid_rows(tmx) * 128; }
constexpr int mid_kb_max(int tmx) { return 64 / tmx; }

struct MidArgs {
  GemmArgs g;
  int kb_per_split, splits, n_chunks;  // n_chunks = ceil(N / (16 * RG))
  float* partials;                     // [n_chunks][splits][RG * TMX][64 lanes] x 4 floats
  unsigned int* counters;              // one per chunk
  int64_t partials_per_entry;          // floats; a batch (g.batch > 1, entry = blockIdx.z) keeps one such array and n_chunks counters per entry
};

template <int RG>
struct WUnit {  // one K-block of a wavefront's weight rows in MFMA operand layout, and its weight-block scale
  u32x4 lo[RG], hi[RG];
  float ws;
};

__device__ __forceinline__ v8i join8(u32x4 lo, u32x4 hi) {
  v8i f;
  f[0] = (int)lo.x; f[1] = (int)lo.y; f[2] = (int)lo.z; f[3] = (int)lo.w;
  f[4] = (int)hi.x; f[5] = (int)hi.y; f[6] = (int)hi.z; f[7] = (int)hi.w;
  return f;
}

template <int TMX, int RG, int WAVES, int DEPTH, int MODE>
__global__ __launch_bounds__(WAVES * 64) void fp8_gemm_midm_kernel(MidArgs a) {
  constexpr int NT = WAVES * 64;
  constexpr int kMidRows = mid_rows(TMX), kMidStageBytes = mid_stage_bytes(TMX);
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];  // [kb][64 rows][128 B], then As [kb][64]
  if (a.g.batch > 1) {  // uniform: this workgroup's entry of the batch
    const int64_t z = blockIdx.z;
    a.g.X += z * a.g.x_batch_bytes;
    a.g.W += z * a.g.w_batch_bytes;
    a.g.C = reinterpret_cast<uint8_t*>(a.g.C) + z * a.g.c_batch_bytes;
    a.g.xs += z * a.g.xs_batch_stride;
    a.g.ws += z * a.g.ws_batch_stride;
    if (a.partials) a.partials += z * a.partials_per_entry;
    if (a.counters) a.counters += z * a.n_chunks;
    if (a.g.last_entry_rows > 0 && z == a.g.batch - 1) a.g.M = a.g.last_entry_rows;
  }
  const GemmArgs& g = a.g;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, lg = lane >> 4;
  const int split = (int)blockIdx.y;
  const int kb0 = split * a.kb_per_split;
  const int kbs = (g.KB - kb0 < a.kb_per_split) ? g.KB - kb0 : a.kb_per_split;  // >= 1: splits = ceil(KB / kb_per_split)
  const int chunk = (int)blockIdx.x * WAVES + wave;
  const bool active = chunk < a.n_chunks;  // uniform over the wavefront
  const int n0 = active ? chunk * 16 * RG : 0;

  // this lane's weight rows (rows past the edge alias the last valid row; never stored)
  const uint8_t* wrow[RG];
#pragma unroll
  for (int r = 0; r < RG; ++r) {
    int n = n0 + r * 16 + l16;
    n = n < g.N ? n : g.N - 1;
    wrow[r] = g.W + (int64_t)n * g.ldw + (int64_t)kb0 * 128 + lg * 16;
  }
  const float* const ws_ptr =
      (MODE == kModeBlock) ? uniform_ptr(g.ws + (int64_t)(n0 >> 7) * g.ws_rs + (int64_t)kb0 * g.ws_cs) : nullptr;
  auto load_unit = [&](WUnit<RG>& u, int k) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      u.lo[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[r] + (int64_t)k * 128));
      u.hi[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[r] + (int64_t)k * 128 + 64));
    }
    u.ws = (MODE == kModeBlock) ? ws_ptr[(int64_t)k * g.ws_cs] : 1.f;
  };

  // the first DEPTH K-blocks of weights are on their way while the activations are staged
  WUnit<RG> ring[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (active && d < kbs) load_unit(ring[d], d);

  // ---- activations of this block's K range -> LDS: row R, logical 16-byte chunk c at R * 128 + ((c ^ (R & 7)) << 4).
  // Direct global -> LDS loads (no registers, nothing to wait for until the barrier): one instruction moves a
  // slab of 8 rows x 128 bytes, lane L landing at byte 16 L of the slab, i.e. row L >> 3, physical chunk L & 7; the
  // lane therefore fetches logical chunk (L & 7) ^ (row & 7) of its row.  Wavefront w takes the slabs w, w + WAVES, ...
  {
    constexpr int kSlabs = 2 * TMX;                          // per K-block
    constexpr int kPer = (kSlabs + WAVES - 1) / WAVES;       // slabs per wavefront and K-block (some wavefronts none)
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    uint32_t xoff[kPer];
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      const int row = (wave + i * WAVES) * 8 + (lane >> 3);
      const int src = row < g.M ? row : g.M - 1;
      xoff[i] = (uint32_t)src * (uint32_t)g.ldx + (uint32_t)((((lane & 7) ^ ((lane >> 3) & 7))) << 4);  // ldx < 2^23
    }
    const uint8_t* const xbase = uniform_ptr(g.X + (int64_t)kb0 * 128);
    for (int kb = 0; kb < kbs; ++kb) {
#pragma unroll
      for (int i = 0; i < kPer; ++i) {
        if (wave + i * WAVES < kSlabs) {  // uniform over the wavefront
          const uint8_t* const src = xbase + (int64_t)kb * 128;
          const uint32_t dst = lds_base + (uint32_t)(kb * kMidStageBytes + (wave + i * WAVES) * 1024);
          asm volatile("s_mov_b32 m0, %2\n\t"
                       "s_nop 0\n\t"
                       "global_load_lds_dwordx4 %0, %1"
                       :
                       : "v"(xoff[i]), "s"(src), "s"(dst)
                       : "memory", "m0");
        }
      }
    }
  }
  float* const xs_lds = reinterpret_cast<float*>(lds + a.kb_per_split * kMidStageBytes);
  if (MODE == kModeBlock) {
    for (int i = tid; i < kbs * kMidRows; i += NT) {
      const int kb = i / kMidRows, row = i % kMidRows;
      const int src = row < g.M ? row : g.M - 1;
      xs_lds[i] = g.xs[(int64_t)src * g.xs_rs + (int64_t)(kb0 + kb) * g.xs_cs];
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // the direct loads are not tracked by the compiler
  __syncthreads();
  if (!active) return;  // no barrier below

  v4f acc[RG][TMX];
#pragma unroll
  for (int r = 0; r < RG; ++r)
#pragma unroll
    for (int t = 0; t < TMX; ++t) acc[r][t] = v4f{0.f, 0.f, 0.f, 0.f};

  // fragment of the 16-row group t for this lane: row t * 16 + l16, logical chunks lg and lg + 4
  const int frag_off = l16 * 128 + ((lg ^ (l16 & 7)) << 4);
  // the ring index is static: the body is written out once per register set
  int kb = 0;
  while (kb < kbs) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (kb < kbs) {
        WUnit<RG>& u = ring[d];
        const uint8_t* const xt = lds + kb * kMidStageBytes;
        v8i xf[TMX];
        float sc[TMX];
#pragma unroll
        for (int t = 0; t < TMX; ++t) {
          const u32x4 lo = *reinterpret_cast<const u32x4*>(xt + t * 2048 + frag_off);
          const u32x4 hi = *reinterpret_cast<const u32x4*>(xt + t * 2048 + (frag_off ^ 64));
          xf[t] = join8(lo, hi);
          sc[t] = (MODE == kModeBlock) ? xs_lds[kb * kMidRows + t * 16 + l16] * u.ws : 1.f;
        }
#pragma unroll
        for (int r = 0; r < RG; ++r) {
          const v8i wf = join8(u.lo[r], u.hi[r]);
#pragma unroll
          for (int t = 0; t < TMX; ++t) {
            if (MODE == kModeBlock) {
              const v4f p = mfma_fp8_16x16x128(wf, xf[t], v4f{0.f, 0.f, 0.f, 0.f});
              acc[r][t][0] = __builtin_fmaf(p[0], sc[t], acc[r][t][0]);
              acc[r][t][1] = __builtin_fmaf(p[1], sc[t], acc[r][t][1]);
              acc[r][t][2] = __builtin_fmaf(p[2], sc[t], acc[r][t][2]);
              acc[r][t][3] = __builtin_fmaf(p[3], sc[t], acc[r][t][3]);
            } else {
              acc[r][t] = MODE == kModeRowColI8 ? mfma_i8_16x16x128(wf, xf[t], acc[r][t]) : mfma_fp8_16x16x128(wf, xf[t], acc[r][t]);
            }
          }
        }
        if (kb + DEPTH < kbs) load_unit(u, kb + DEPTH);
        ++kb;
      }
    }
  }

  // ---- K split over blocks: publish, count in, and let the wavefront that arrives last add the splits in order
  if (a.splits > 1) {
    constexpr int kSlotFloats = RG * TMX * 64 * 4;
    const uint32_t l_off = (uint32_t)lane * 16u;
    float* const mine = uniform_ptr(a.partials + ((size_t)chunk * a.splits + split) * kSlotFloats);
#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
      for (int t = 0; t < TMX; ++t) store_x4_agent(mine + (r * TMX + t) * 256, l_off, acc[r][t]);
    wait_vmem_all();
    unsigned int* const cnt = a.counters + chunk;
    unsigned int prev = 0;
    if (lane == 0) prev = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    prev = (unsigned int)__builtin_amdgcn_readfirstlane((int)prev);
    if (prev != (unsigned int)(a.splits - 1)) return;
    // The splits' sums are fetched kBatch splits at a time (one round trip to memory per batch instead of one per
    // split) and added one split after the other, in split order.  Every batch is loaded, waited for and consumed
    // inside one iteration: the loads are not tracked by the compiler, so no register may be in flight across the
    // loop's back edge.
    constexpr int kBatch = RG * TMX <= 8 ? 4 : 2;
    for (int s0 = 0; s0 < a.splits; s0 += kBatch) {
      v4f tmp[kBatch][RG][TMX];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        const int s = s0 + b < a.splits ? s0 + b : a.splits - 1;  // past the end: re-read the last split, unused
        const float* const src = uniform_ptr(a.partials + ((size_t)chunk * a.splits + s) * kSlotFloats);
#pragma unroll
        for (int r = 0; r < RG; ++r)
#pragma unroll
          for (int t = 0; t < TMX; ++t) load_x4_agent(tmp[b][r][t], src + (r * TMX + t) * 256, l_off);
      }
#pragma unroll
      for (int b = 0; b < kBatch; ++b)  // the values are operands of the wait, so no use can move above it
#pragma unroll
        for (int r = 0; r < RG; ++r)
#pragma unroll
          for (int t = 0; t < TMX; ++t) asm volatile("s_waitcnt vmcnt(0)" : "+v"(tmp[b][r][t]) : : "memory");
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        if (s0 + b < a.splits) {
#pragma unroll
          for (int r = 0; r < RG; ++r)
#pragma unroll
            for (int t = 0; t < TMX; ++t) {
              // (no "0 + x" in the sum; int8 operands: the registers hold int32 sums, added as such)
              if (s0 + b == 0) acc[r][t] = tmp[b][r][t];
              else if (MODE == kModeRowColI8) acc[r][t] = __builtin_bit_cast(v4f, __builtin_bit_cast(v4i, acc[r][t]) + __builtin_bit_cast(v4i, tmp[b][r][t]));
              else acc[r][t] += tmp[b][r][t];
            }
        }
      }
    }
    if (lane == 0) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
  }

  // ---- results: the lane holds m = t * 16 + l16, n = n0 + r * 16 + 4 * lg + [0, 4)
#pragma unroll
  for (int t = 0; t < TMX; ++t) {
    const int m = t * 16 + l16;
    if (m >= g.M) continue;
#pragma unroll
    for (int r = 0; r < RG; ++r) store_output4<MODE>(g, m, n0 + r * 16 + lg * 4, acc[r][t]);
  }
}

template <int TMX, int RG, int WAVES, int DEPTH>
int launch_mid(const MidArgs& ma, int mode, hipStream_t stream) {
  constexpr int kPerKb = mid_stage_bytes(TMX) + mid_rows(TMX) * 4;
  const int lds_bytes = ma.kb_per_split * kPerKb;
  auto kb = fp8_gemm_midm_kernel<TMX, RG, WAVES, DEPTH, kModeBlock>;
  auto kr = fp8_gemm_midm_kernel<TMX, RG, WAVES, DEPTH, kModeRowCol>;
  auto ki = fp8_gemm_midm_kernel<TMX, RG, WAVES, DEPTH, kModeRowColI8>;
  static PerDeviceFlags lds_limit_raised = {};  // per instantiation
  {
    constexpr int kMax = mid_kb_max(TMX) * kPerKb;
    const hipError_t e = raise_dynamic_lds_limit(lds_limit_raised, kMax, reinterpret_cast<const void*>(kb), reinterpret_cast<const void*>(kr),
                                                  reinterpret_cast<const void*>(ki));
    if (e != hipSuccess) FG_FAIL(FG_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", kMax, hipGetErrorString(e));
  }
  const dim3 grid((uint32_t)ceil_div(ma.n_chunks, WAVES), (uint32_t)ma.splits, (uint32_t)(ma.g.batch > 1 ? ma.g.batch : 1)), block(WAVES * 64);
  if (mode == kModeBlock) FG_LAUNCH(kb, grid, block, lds_bytes, stream, ma);
  else if (mode == kModeRowColI8) FG_LAUNCH(ki, grid, block, lds_bytes, stream, ma);
  else FG_LAUNCH(kr, grid, block, lds_bytes, stream, ma);
  FG_CHECK_LAUNCH("fp8_gemm_midm_kernel");
  return FG_OK;
}

}  // namespace

MidMPlan plan_mid_m(int64_t M, int64_t N, int64_t K, int64_t entries) {
  MidMPlan p = {};
  if (entries < 1) entries = 1;  // equal problems launched together: their wavefronts fill the GPU together
  // (16- and 32-row variants of this kernel were measured against the decode kernels: the 16-row one slower on every shape;
  // the 32-row one ahead from 21 rows against narrow weights with long K -- N = 2112, K = 7168, M = 24 / 32: 11.9 / 14.0 -> 10.7 / 10.8 us --
  // until the decode kernels took 17..32 rows in two parts of up to 16: 7.7 / 9.2 us)
  if (M <= 32 || M > 128 || N < 1 || K < 128 || K % 128 != 0) return p;
  const int64_t KB = K / 128;
  // 33..48 rows stage 48: a quarter less LDS per K-block (21 fit), MFMA work and partial sums: 2-8 % faster than with 64 rows
  // on 13 of 14 shapes (M = 40: N = 7168, K = 16384: 40.2 -> 37.0 us; N = 2112, K = 7168: 13.0 -> 12.2; N = 4096, K = 14336: 22.4 -> 21.1;
  // N = 14336, K = 4096: 20.8 -> 21.1)
  // (80 and 96 rows staged for 65..96 rows do not soften the step to the tile kernel at 65 rows: M = 80, N = 2112, K = 7168:
  // 19.4 us there, 19.1 here; N = 7168, K = 16384: 40 against 58; N = K = 4096: 16.2 against 15.8; N = 24576, K = 1536: 14.8 against 17.7)
  const int tmx = M <= 48 ? 3 : M <= 64 ? 4 : 8;
  const int64_t kb_max = mid_kb_max(tmx);
  const int64_t min_splits = ceil_div(KB, kb_max);
  int rg;
  int64_t splits;
  if (tmx <= 4) {
    // Measured on the DeepSeek-V3 shapes with 64 rows (weights rotated through 512 MB): the narrowest row group
    // wins almost everywhere (more wavefronts, each with 16 KB of weights in flight); K is split until there are
    // ~1800 wavefronts but not below 8 K-blocks per block (every split writes and reads N x 64 fp32 sums: +50 % of
    // the weight bytes at 8 K-blocks, +25 % at 16), and never less than LDS requires.
    rg = 1;
    if (ceil_div(N, 16) * entries * min_splits >= 3000) rg = 2;  // plenty of wavefronts: N = 7168, K = 16384: 43 -> 39 us
    splits = ceil_div((int64_t)1800, ceil_div(N, 16 * rg) * entries);
    const int64_t max_splits = KB / 8 > min_splits ? KB / 8 : min_splits;
    splits = splits < min_splits ? min_splits : (splits > max_splits ? max_splits : splits);
  } else {
    // 65..128 rows: a K-block of activations is 16 KB, so LDS holds 8 and every split costs as many bytes as the
    // weights of 8 K-blocks.  Measured (M = 128): one row group per wavefront beats two wherever this kernel
    // beats the tile kernel at all, which is for weights of up to ~28 MB (see the caller's rule).
    rg = 1;
    splits = min_splits;
  }
  while (rg < 4 && ceil_div(N, 16 * rg) > FG_WORKSPACE_COUNTER_BYTES / 4) rg <<= 1;
  if (tmx == 8 && rg > 2) return p;
  if (tmx <= 4 && entries == 1 && ceil_div(N, 128) > cu_count()) {
    // Weights too wide for the tile kernel's one round of 128 x 128 tiles run in several rounds of blocks here, and the
    // wavefront count above says nothing about how full the last round is.  Take the split with the least
    // rounds x (K-blocks per block + 2, + 4 with K split) instead (2: staging; 4: a block's partial sums, written and read
    // back, are as many bytes as four K-blocks of its weights; N = 57344, K = 8192: eight ranges fill seven rounds exactly and
    // take 150 us, four ranges in four rounds 134 us).  M = 64:
    // N = 49152, K = 2048: two ranges, 768 blocks on 512 places, 40.5 us -> one range, 192 blocks, 29.9 us; N = 37888,
    // K = 3584: two ranges, 296 blocks on 256 places, 58.4 -> three, 444 blocks, 49.5 us; M = 48: N = 40960, K = 5120: 84.4 -> 67.6 us;
    // N = 152064, K = 3584: 163.5 -> 147.9 us.
    const int64_t max_splits = KB / 8 > min_splits ? KB / 8 : min_splits;
    const int64_t per_kb = mid_stage_bytes(tmx) + mid_rows(tmx) * 4;
    int64_t best = splits, best_cost = 0;
    for (int64_t s = min_splits; s <= max_splits; ++s) {
      const int64_t kb_s = ceil_div(KB, s), s_eff = ceil_div(KB, kb_s);
      const int64_t waves = kb_s * per_kb > 80 * 1024 ? 8 : 4;
      const int64_t blocks = ceil_div(ceil_div(N, 16 * rg), waves) * s_eff;
      const int64_t rounds = ceil_div(blocks, (int64_t)cu_count() * (waves == 8 ? 1 : 2));
      const int64_t cost = rounds * (kb_s + 2 + (s_eff > 1 ? 4 : 0));
      if (best_cost == 0 || cost < best_cost) { best = s_eff; best_cost = cost; }
    }
    splits = best;
  }
  const int64_t kbps = ceil_div(KB, splits);
  splits = ceil_div(KB, kbps);
  p.tmx = tmx;
  p.rg = rg;
  p.kb_per_split = (int)kbps;
  p.splits = (int)splits;
  p.n_chunks = (int)ceil_div(N, 16 * rg);
  if (p.n_chunks > FG_WORKSPACE_COUNTER_BYTES / 4 || splits > 65535) return p;
  // one block per compute unit when its activations take more than half of LDS: then it should bring 8 wavefronts
  p.waves = kbps * (mid_stage_bytes(tmx) + mid_rows(tmx) * 4) > 80 * 1024 ? 8 : 4;
  p.workspace_bytes = splits > 1 ? (size_t)FG_WORKSPACE_COUNTER_BYTES + (size_t)p.n_chunks * splits * rg * tmx * 64 * 16 : 0;
  p.use = true;
  return p;
}

int launch_mid_m(const GemmArgs& g, int mode, const MidMPlan& plan, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  MidArgs ma;
  ma.g = g;
  ma.kb_per_split = plan.kb_per_split;
  ma.splits = plan.splits;
  ma.n_chunks = plan.n_chunks;
  ma.partials = nullptr;
  ma.counters = nullptr;
  ma.partials_per_entry = 0;
  if (plan.splits > 1) {
    const size_t entries = g.batch > 1 ? (size_t)g.batch : 1;
    const size_t per_entry = plan.workspace_bytes - FG_WORKSPACE_COUNTER_BYTES;
    const size_t need = FG_WORKSPACE_COUNTER_BYTES + entries * per_entry;
    ma.partials_per_entry = (int64_t)(per_entry / sizeof(float));
    if (entries * (size_t)plan.n_chunks * sizeof(unsigned int) > FG_WORKSPACE_COUNTER_BYTES)
      FG_FAIL(FG_ERR_WORKSPACE, "fp8 gemm (33..128 rows): %zu batch entries of %d chunks do not fit the counter area", entries, plan.n_chunks);
    if (!workspace || workspace_bytes < need)
      FG_FAIL(FG_ERR_WORKSPACE, "fp8 gemm (33..128 rows): workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    if ((uintptr_t)workspace % 16 != 0) FG_FAIL(FG_ERR_INVALID_ARG, "fp8 gemm (33..128 rows): workspace must be 16-byte aligned");
    ma.counters = reinterpret_cast<unsigned int*>(workspace);
    ma.partials = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + FG_WORKSPACE_COUNTER_BYTES);
  }
  if (plan.tmx == 8) {
    if (plan.rg == 2) return plan.waves == 8 ? launch_mid<8, 2, 8, 4>(ma, mode, stream) : launch_mid<8, 2, 4, 4>(ma, mode, stream);
    return plan.waves == 8 ? launch_mid<8, 1, 8, 8>(ma, mode, stream) : launch_mid<8, 1, 4, 8>(ma, mode, stream);
  }
  if (plan.tmx == 3) {
    if (plan.rg == 4) return plan.waves == 8 ? launch_mid<3, 4, 8, 2>(ma, mode, stream) : launch_mid<3, 4, 4, 2>(ma, mode, stream);
    if (plan.rg == 2) return plan.waves == 8 ? launch_mid<3, 2, 8, 4>(ma, mode, stream) : launch_mid<3, 2, 4, 4>(ma, mode, stream);
    return plan.waves == 8 ? launch_mid<3, 1, 8, 8>(ma, mode, stream) : launch_mid<3, 1, 4, 8>(ma, mode, stream);
  }
  if (plan.rg == 4) return plan.waves == 8 ? launch_mid<4, 4, 8, 2>(ma, mode, stream) : launch_mid<4, 4, 4, 2>(ma, mode, stream);
  if (plan.rg == 2) return plan.waves == 8 ? launch_mid<4, 2, 8, 4>(ma, mode, stream) : launch_mid<4, 2, 4, 4>(ma, mode, stream);
  return plan.waves == 8 ? launch_mid<4, 1, 8, 8>(ma, mode, stream) : launch_mid<4, 1, 4, 8>(ma, mode, stream);
}

}  // namespace fg
