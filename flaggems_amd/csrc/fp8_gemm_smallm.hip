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
};

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

template <int TMX, int WAVES, int MODE>
__global__ __launch_bounds__(WAVES * 64) void fp8_gemm_smallm_kernel(SmallArgs a) {
  constexpr int NT = WAVES * 64;
  constexpr int MROWS = 16 * TMX;
  __shared__ float red[WAVES][MROWS][kChunkRows];  // 4 KB * TMX per wavefront
  __shared__ int last_flag;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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

  // ---- add the wavefronts' results in LDS: lane holds m = t*16 + l16, n = r*16 + 4*lg + [0,4)
#pragma unroll
  for (int r = 0; r < kRowGroups; ++r)
#pragma unroll
    for (int t = 0; t < TMX; ++t)
      *reinterpret_cast<v4f*>(&red[wave][t * 16 + l16][r * 16 + lg * 4]) = acc[r][t];
  __syncthreads();

  constexpr int kOut = MROWS * kChunkRows;
  if (a.splits == 1) {
    for (int i = tid; i < kOut; i += NT) {
      const int m = i / kChunkRows, nn = i % kChunkRows;
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) v += red[w][m][nn];
      if (m < g.M && n0 + nn < g.N) store_output<MODE>(g, m, n0 + nn, v);
    }
    return;
  }

  // ---- split K: publish this block's partial tile, last arriver reduces in split order
  float* const mine = a.partials + ((int64_t)chunk * a.splits + split) * kOut;
  for (int i = tid; i < kOut; i += NT) {
    const int m = i / kChunkRows, nn = i % kChunkRows;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) v += red[w][m][nn];
    // device-scope store: written through to memory, where blocks on other XCDs (own L2 each) read it
    __hip_atomic_store(mine + i, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // A device-scope fence here would write back and invalidate the whole L2 (measured ~50 us per
  // launch).  The partial tiles bypass the L2 on both sides instead, so it is enough that every
  // store of this block has been acknowledged before the counter moves.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (tid == 0) {
    const unsigned int prev = __hip_atomic_fetch_add(&a.counters[chunk], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last_flag = (prev == (unsigned int)(a.splits - 1)) ? 1 : 0;
  }
  __syncthreads();
  if (!last_flag) return;
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

template <int TMX, int WAVES>
int launch_t(const SmallArgs& sa, int mode, hipStream_t stream) {
  const dim3 grid((uint32_t)(sa.n_chunks * sa.splits)), block(WAVES * 64);
  if (mode == kModeBlock) hipLaunchKernelGGL((fp8_gemm_smallm_kernel<TMX, WAVES, kModeBlock>), grid, block, 0, stream, sa);
  else hipLaunchKernelGGL((fp8_gemm_smallm_kernel<TMX, WAVES, kModeRowCol>), grid, block, 0, stream, sa);
  FG_CHECK_LAUNCH("fp8_gemm_smallm_kernel");
  return FG_OK;
}

}  // namespace

SmallMPlan plan_small_m(int64_t M, int64_t N, int64_t K) {
  SmallMPlan p = {};
  p.use = false;
  if (M < 1 || M > 64 || N < 1 || K < 128 || K % 128 != 0) return p;
  p.tmx = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  p.waves = p.tmx == 4 ? 4 : 8;  // LDS reduction buffer is 4 KB * tmx per wavefront
  p.n_chunks = (int)ceil_div(N, kChunkRows);
  if (p.n_chunks > FG_WORKSPACE_COUNTER_BYTES / 4) return p;
  const int64_t KB = K / 128;
  // aim for ~8 wavefronts per CU on 256 CUs, each with at least one K-block
  const int64_t units = (int64_t)p.n_chunks * KB;
  int64_t kpw = units / 2048;
  if (kpw < 1) kpw = 1;
  int64_t splits = ceil_div(KB, kpw * p.waves);
  if (splits < 1) splits = 1;
  // partial tiles cost 2 * splits * 16*tmx * 64 * 4 bytes per chunk against 64 * K weight bytes: keep
  // them under a quarter of the weight traffic
  const int64_t max_splits = K / (32 * 16 * p.tmx) > 1 ? K / (32 * 16 * p.tmx) : 1;
  if (splits > max_splits) splits = max_splits;
  kpw = ceil_div(KB, splits * p.waves);  // even out
  // a block with idle wavefronts wastes launch slots: fewer wavefronts when K is short
  if (splits == 1 && KB <= 4) { p.waves = 4; kpw = ceil_div(KB, 4); }
  p.kpw = (int)kpw;
  p.splits = (int)splits;
  p.workspace_bytes = splits > 1
      ? (size_t)FG_WORKSPACE_COUNTER_BYTES + (size_t)p.n_chunks * splits * 16 * p.tmx * kChunkRows * sizeof(float)
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
  if (plan.splits > 1) {
    if (!workspace || workspace_bytes < plan.workspace_bytes)
      FG_FAIL(FG_ERR_WORKSPACE, "fp8 gemm (small M): workspace of %zu bytes needed, %zu given", plan.workspace_bytes,
              workspace_bytes);
    if ((uintptr_t)workspace % 16 != 0) FG_FAIL(FG_ERR_INVALID_ARG, "fp8 gemm (small M): workspace must be 16-byte aligned");
    sa.counters = reinterpret_cast<unsigned int*>(workspace);
    sa.partials = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + FG_WORKSPACE_COUNTER_BYTES);
  }
  if (plan.tmx == 1) return plan.waves == 8 ? launch_t<1, 8>(sa, mode, stream) : launch_t<1, 4>(sa, mode, stream);
  if (plan.tmx == 2) return plan.waves == 8 ? launch_t<2, 8>(sa, mode, stream) : launch_t<2, 4>(sa, mode, stream);
  return launch_t<4, 4>(sa, mode, stream);
}

}  // namespace fg
