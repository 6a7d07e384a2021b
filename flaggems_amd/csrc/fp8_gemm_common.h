// Pieces shared by the FP8 GEMM kernels: argument block, conversions, per-element epilogue.
#pragma once

#include "fg_common.h"

namespace fg {

// kModeRowColI8: int8 operands, int32 sums (kept as bit patterns in the fp32 accumulator registers), scales and
// bias as kModeRowCol.
// kModeRowColBF16 / kModeRowColF16 (persistent kernel only): bf16 / fp16 operands, whose rows the kernels take as
// bytes (a 128-byte K-block is 64 elements); row and column scales, and the bias is added in fp32 before the one
// rounding, as aten::_scaled_mm's generic kernel does (src/flag_gems/ops/scaled_mm.py:37-133).
enum { kModeBlock = 0, kModeRowCol = 1, kModeRowColI8 = 2, kModeRowColBF16 = 3, kModeRowColF16 = 4 };

struct GemmArgs {
  const uint8_t* X;  // activations [M, K]
  const uint8_t* W;  // weights [N, K]
  void* C;
  const float* xs;   // block: As [M, KB]; rowcol: a_scale
  const float* ws;   // block: Bs [NB, KB]; rowcol: b_scale
  const void* bias;
  int64_t ldx, ldw, ldc;
  int64_t xs_rs, xs_cs, ws_rs, ws_cs;
  int M, N, K, KB;
  int tiles_m, tiles_n;
  int c_dtype, bias_dtype;
  int xs_per_row, ws_per_col;
  // block mode: the caller guarantees that every scale is a power of two (only the persistent kernel makes use of it)
  int scales_pow2;
  // tile kernel with K split over blocks (fp8_gemm.hip): block b computes K-blocks
  // [split * kb_per_split, ...) of tile b % tiles, split = b / tiles
  int splits, kb_per_split;
  float* split_partials;
  unsigned int* split_counters;
  // tile kernel over a batch of equal problems in one launch: blockIdx.y is the batch entry, whose operands lie
  // these many bytes (X, W, C) or floats (xs, ws) after the previous entry's; batch <= 1: one problem
  int batch;
  int64_t x_batch_bytes, w_batch_bytes, c_batch_bytes, xs_batch_stride, ws_batch_stride;
  // a batch with K split over blocks: every entry has tiles x splits partial tiles of its own, these many floats in
  // all, and tiles x wavefronts counters
  int64_t split_partials_per_entry;
  // staged-activation kernel over equal parts of a lone problem's rows (the entries of a batch that shares the weights):
  // rows of the last part when it has fewer than M, else 0
  int last_entry_rows;
  // decode kernels over parts of a lone problem's rows: the last entry starts this much before where the batch strides
  // would put it, so that it ends with the last row (bytes of X, bytes of C, floats of xs; 0 otherwise)
  int64_t last_x_back_bytes, last_c_back_bytes, last_xs_back;
};

// s_waitcnt vmcnt(0) with expcnt/lgkmcnt left at their maxima (gfx9 encoding)
__device__ __forceinline__ void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return bits_to_float((uint32_t)b << 16); }

__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = float_to_bits(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);  // quiet NaN
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float load_as_float(const void* p, int64_t i, int dtype) {
  if (dtype == FG_F32) return reinterpret_cast<const float*>(p)[i];
  if (dtype == FG_F16) return (float)reinterpret_cast<const _Float16*>(p)[i];
  return bf16_bits_to_float(reinterpret_cast<const uint16_t*>(p)[i]);
}


// Final value of one output element: row/column scaling (row/column mode only), rounding to the
// output type and the bias added after that rounding, in the output type, as the reference's epilogue
// does (src/flag_gems/fused/cutlass_scaled_mm.py:288-305).
template <int MODE>
__device__ __forceinline__ void store_output(const GemmArgs& a, int m, int n, float v) {
  if (MODE == kModeRowColI8) v = (float)__float_as_int(v);  // int8 operands: v carries the bits of an int32 sum
  if (MODE != kModeBlock) v = (v * a.xs[a.xs_per_row ? m : 0]) * a.ws[a.ws_per_col ? n : 0];
  const bool has_bias = (MODE != kModeBlock) && a.bias != nullptr;
  const int64_t off = (int64_t)m * a.ldc + n;
  if (a.c_dtype == FG_BF16) {
    uint16_t h = float_to_bf16_bits(v);
    if (has_bias) h = float_to_bf16_bits(bf16_bits_to_float(h) + load_as_float(a.bias, n, a.bias_dtype));
    reinterpret_cast<uint16_t*>(a.C)[off] = h;
  } else if (a.c_dtype == FG_F16) {
    _Float16 h = (_Float16)v;
    if (has_bias) h = (_Float16)((float)h + load_as_float(a.bias, n, a.bias_dtype));
    reinterpret_cast<_Float16*>(a.C)[off] = h;
  } else if (a.c_dtype == FG_F32) {
    if (has_bias) v = v + load_as_float(a.bias, n, a.bias_dtype);
    reinterpret_cast<float*>(a.C)[off] = v;
  } else {  // FG_FP8_E4M3FN
    uint32_t code = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(v, 0.f, 0, false) & 0xFFu;
    if (has_bias) {
      const float back = __builtin_amdgcn_cvt_f32_fp8((int)code, 0);
      code = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(back + load_as_float(a.bias, n, a.bias_dtype), 0.f, 0, false) & 0xFFu;
    }
    reinterpret_cast<uint8_t*>(a.C)[off] = (uint8_t)code;
  }
}

// Four consecutive columns n .. n + 3 of row m (the four results a lane holds of a 16 x 16 MFMA tile): the same
// arithmetic as store_output, element by element, with the scales of the row/column modes loaded once and one
// 8- or 16-byte store where the four columns exist and the address allows it.
template <int MODE>
__device__ __forceinline__ void store_output4(const GemmArgs& a, int m, int n, v4f acc4) {
  if (n >= a.N) return;
  constexpr bool kRowCol = MODE != kModeBlock;
  float v[4] = {acc4[0], acc4[1], acc4[2], acc4[3]};
  if (MODE == kModeRowColI8) {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = (float)__float_as_int(v[e]);  // int32 sums
  }
  const int nv = (a.N - n < 4) ? a.N - n : 4;
  float bias[4] = {0.f, 0.f, 0.f, 0.f};
  const bool has_bias = kRowCol && a.bias != nullptr;
  if (kRowCol) {
    const float sa = a.xs[a.xs_per_row ? m : 0];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int ne = (e < nv) ? n + e : n;
      v[e] = (v[e] * sa) * a.ws[a.ws_per_col ? ne : 0];
      if (has_bias) bias[e] = load_as_float(a.bias, ne, a.bias_dtype);
    }
  }
  const int64_t off = (int64_t)m * a.ldc + n;
  if (a.c_dtype == FG_BF16) {
    uint16_t h[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      h[e] = float_to_bf16_bits(v[e]);
      if (has_bias) h[e] = float_to_bf16_bits(bf16_bits_to_float(h[e]) + bias[e]);
    }
    uint16_t* const cp = reinterpret_cast<uint16_t*>(a.C) + off;
    if (nv == 4 && ((uintptr_t)cp % 8 == 0)) {
      *reinterpret_cast<u32x2*>(cp) = u32x2{(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
    } else {
      for (int e = 0; e < nv; ++e) cp[e] = h[e];
    }
  } else if (a.c_dtype == FG_F16) {
    uint16_t h[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      _Float16 f = (_Float16)v[e];
      if (has_bias) f = (_Float16)((float)f + bias[e]);
      h[e] = __builtin_bit_cast(uint16_t, f);
    }
    uint16_t* const cp = reinterpret_cast<uint16_t*>(a.C) + off;
    if (nv == 4 && ((uintptr_t)cp % 8 == 0)) {
      *reinterpret_cast<u32x2*>(cp) = u32x2{(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
    } else {
      for (int e = 0; e < nv; ++e) cp[e] = h[e];
    }
  } else if (a.c_dtype == FG_F32) {
    float* const cp = reinterpret_cast<float*>(a.C) + off;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = has_bias ? v[e] + bias[e] : v[e];
    if (nv == 4 && ((uintptr_t)cp % 16 == 0)) {
      *reinterpret_cast<v4f*>(cp) = v4f{v[0], v[1], v[2], v[3]};
    } else {
      for (int e = 0; e < nv; ++e) cp[e] = v[e];
    }
  } else {  // FG_FP8_E4M3FN
    uint8_t* const cp = reinterpret_cast<uint8_t*>(a.C) + off;
    for (int e = 0; e < nv; ++e) {
      uint32_t code = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(v[e], 0.f, 0, false) & 0xFFu;
      if (has_bias) {
        // the reference adds the bias to the already rounded output, in the output type
        const float back = __builtin_amdgcn_cvt_f32_fp8((int)code, 0);
        code = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(back + bias[e], 0.f, 0, false) & 0xFFu;
      }
      cp[e] = (uint8_t)code;
    }
  }
}

__device__ __forceinline__ v4f mfma_fp8_16x16x128(v8i a, v8i b, v4f c) {
  // cbsz = blgp = 0: both operands e4m3; zero scale operands select the unscaled instruction
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

// One K-block (128) of int8 products into int32 sums: two 16x16x64 instructions, each on the half of the fragment
// registers that holds the same K positions in both operands (the operands share one K layout, whatever it is).
__device__ __forceinline__ v4f mfma_i8_16x16x128(v8i a, v8i b, v4f c) {
  v4i acc = __builtin_bit_cast(v4i, c);
  const v4i a_lo = {a[0], a[1], a[2], a[3]}, a_hi = {a[4], a[5], a[6], a[7]};
  const v4i b_lo = {b[0], b[1], b[2], b[3]}, b_hi = {b[4], b[5], b[6], b[7]};
  acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_lo, b_lo, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_hi, b_hi, acc, 0, 0, 0);
  return __builtin_bit_cast(v4f, acc);
}

// Operands of inline assembly with an "s" constraint must be in scalar registers; this makes the compiler see
// that a (uniform) pointer is.
template <typename T>
__device__ __forceinline__ T* uniform_ptr(T* p) {
  const uint64_t v = (uint64_t)p;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return (T*)(((uint64_t)hi << 32) | lo);
}

// 16-byte accesses that other XCDs can see: written through to memory / read past this XCD's L2 (the same
// cache-control bit the compiler sets for agent-scope atomic loads and stores).  Not tracked by the
// compiler's wait-count insertion: callers wait explicitly.
__device__ __forceinline__ void store_x4_agent(float* base, uint32_t byte_off, const v4f& v) {
  asm volatile("global_store_dwordx4 %0, %1, %2 sc1" : : "v"(byte_off), "v"(v), "s"(base) : "memory");
}
__device__ __forceinline__ void load_x4_agent(v4f& v, const float* base, uint32_t byte_off) {
  asm volatile("global_load_dwordx4 %0, %1, %2 sc1" : "=v"(v) : "v"(byte_off), "s"(base) : "memory");
}


// Compute units of the current device (256 when it cannot be asked, e.g. on a host without a GPU).
int cu_count();

// Small-M (decode) path, fp8_gemm_smallm.hip.  `use` reports whether the kernel takes the problem.
struct SmallMPlan {
  bool use;
  bool staged;    // weight bytes fetched in 256-byte runs (K-block pairs) and transposed through LDS
  int tmx;        // 16-row activation fragments: 1, 2 or 4
  int rg;         // 16-row weight groups per output chunk: 1, 2 or 4
  int q;          // staged: 4-row weight groups the kernel loads per chunk (<= 4 * rg)
  bool xlds;      // staged: the block keeps the activations of its K range in LDS
  bool own;       // staged: every wavefront has a chunk of its own and walks all of K
  bool ring;      // staged, xlds: two slots of activations per wavefront, refilled pair by pair
  int waves;      // wavefronts per block: 4 or 8
  int kpw;        // K-blocks (K-block pairs when staged) per wavefront
  int splits;     // blocks along K that share one 64-row output chunk
  int n_chunks;   // ceil(N / (16 * rg))
  size_t workspace_bytes;
};
// fp8_gemm_anyblock.hip: block-scaled product for scale blocks of any size (a plain fp32 tile kernel).
int launch_anyblock(const GemmArgs& g, int64_t block_n, int64_t block_k, hipStream_t stream);

SmallMPlan plan_small_m(int64_t M, int64_t N, int64_t K, int64_t entries = 1);
int launch_small_m(const GemmArgs& a, int mode, const SmallMPlan& plan, void* workspace, size_t workspace_bytes,
                   hipStream_t stream);


// 33 <= M <= 128 rows, fp8_gemm_midm.hip: activations staged in LDS once per block, weights streamed.
struct MidMPlan {
  bool use;
  int tmx;           // 16-row activation groups staged: 3 (M <= 48), 4 (M <= 64) or 8
  int rg;            // 16-row weight groups per wavefront: 1, 2 or 4
  int waves;         // wavefronts per block: 4 or 8
  int kb_per_split;  // K-blocks per block (<= 16)
  int splits;        // blocks along K
  int n_chunks;      // ceil(N / (16 * rg))
  size_t workspace_bytes;
};
MidMPlan plan_mid_m(int64_t M, int64_t N, int64_t K, int64_t entries = 1);
int launch_mid_m(const GemmArgs& a, int mode, const MidMPlan& plan, void* workspace, size_t workspace_bytes,
                 hipStream_t stream);

// Persistent 256x256 kernel, fp8_gemm_pingpong.hip: bf16 output with 16-byte aligned rows, M > 128 (or M > 64 when
// the workspace lets it share tiles along K);
// the caller has checked that the operands qualify for direct global->LDS loads.
bool pingpong_takes(const GemmArgs& a, int mode, const void* workspace, size_t workspace_bytes);
int launch_pingpong(const GemmArgs& a, int mode, void* workspace, size_t workspace_bytes, hipStream_t stream);
// workspace that lets the persistent kernel split tiles along K between blocks (0: never useful for this shape)
size_t pingpong_workspace_bytes(int64_t M, int64_t N, int64_t K);

// Grouped problem for the persistent kernel: rows [ends[e-1], ends[e]) of X and C (ends[-1] = 0; a device table
// of cumulative int32 ends) meet weight matrix e, w_group_stride bytes and ws_group_stride scale floats after
// matrix 0.  Block scales, bf16 result; a.M is the total row count, a.W / a.ws point at matrix 0.
struct GroupedGemm {
  const int* ends;
  int64_t n_groups;
  int64_t w_group_stride, ws_group_stride;
  // optional gather: row m of the sorted order is row row_index[m] / index_div of X (x_rows rows) and of its scales
  const int* row_index;
  int64_t index_div, x_rows;
  // optional scatter (needs row_index): sorted row m is stored to row row_index[m] of C (c_rows rows; entries outside
  // [0, c_rows) store nothing), multiplied by row_weight[row_index[m]] when row_weight is given; c_rows = 0: row m
  int64_t c_rows;
  const float* row_weight;
};
int launch_grouped(const GemmArgs& a, const GroupedGemm& grouped, void* workspace, size_t workspace_bytes, hipStream_t stream);
// workspace that lets launch_grouped read row-major activation scales from a transposed copy
size_t grouped_workspace_bytes(int64_t M, int64_t K);

}  // namespace fg
