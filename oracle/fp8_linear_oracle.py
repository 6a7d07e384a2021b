"""CPU restatement of the reference's torch implementations of the FP8 quantized
linear path (activation quantizers, 128x128 weight quantizer, block-scaled GEMM,
per-token/per-channel scaled GEMM).

TEST INFRASTRUCTURE. Only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this module.  The product (flaggems_amd) never
imports it and has no CPU fallback.

Every function restates one torch-native reference function that the reference
repository keeps in its test/benchmark files, and cites it.  All functions run
on CPU tensors with plain torch ops; nothing here touches a GPU.

Pinning status (what checks each function against something other than itself;
the checks live in tests/test_oracle_*.py):

* act_quant_ref, per_token_group_quant_fp8_ref, per_token_group_quant_fp8_div_ref,
  per_block_cast_to_fp8_ref, per_token_cast_to_fp8_ref -- pinned by a brute-force
  numpy quantizer built on the bit-level E4M3 encoder of oracle/e4m3.py (itself
  pinned against ``tensor.to(torch.float8_e4m3fn)`` on all 65 536 bf16 patterns
  and against a nearest-value search), by the invariants "max |x| of a group
  encodes to +-448", "codes(-x) = sign-flipped codes(x)", "ue8m0 scale is the
  power of two in [s, 2s)", and by hand-worked special cases (all-zero group,
  NaN, Inf, a lone huge element).
* block_fp8_matmul_dequant_ref, block_fp8_matmul_tiled_ref -- pinned against each
  other (two different algorithms from two reference files), a float64 triple
  loop on tiny shapes, and closed forms (unit scales -> plain matmul, one-hot
  rows pick scaled weight rows exactly, power-of-two scales are exact).
* grouped_block_fp8_matmul_ref -- a loop of block_fp8_matmul_tiled_ref over row
  segments; pinned by the dequantise-then-matmul reference per segment, by "one
  group = the plain GEMM", by "identical weights in every group = the plain GEMM
  whatever the segment ends", and by a float64 loop on a tiny ragged case.
* fp8_block_einsum_ref -- dequantise-then-einsum over [b, h, r] x [h, d, r]; pinned
  per head against block_fp8_matmul_tiled_ref (a different order of operations)
  and by a float64 loop on a tiny case.
* inv_rope_ref, fused_inv_rope_fp8_quant_ref -- the rotation is pinned by known answers the mathematics fixes (a pair
  (cos t, sin t) rotated back by t is (1, 0); forward rotation would give (cos 2t, sin 2t)), by a float64
  evaluation with complex numbers (a different formula), by exact preservation of pair norms at the angles 0, pi/2
  and pi, and by position 0 leaving the input untouched; the quantizer half is pinned by equality with
  per_token_group_quant_fp8_kernel_ref's formulas on the same values (itself pinned by the brute-force quantizer),
  and the layout and packed exponents by inputs whose group maxima are 448 * 2^k, so that scale k and byte 127 + k
  are known in advance (tests/test_oracle_inv_rope.py).
* topk_softmax_ref, grouped_topk_ref -- the reference tests both against vLLM's CUDA operators, which are absent here;
  the restatements follow the reference's own Triton kernels and are pinned by library routines and closed forms:
  torch.softmax + torch.topk on rows without ties, rows of equal logits (experts 0 .. k-1 at 1 / E each), weights that
  sum to 1 after renormalisation, the published DeepSeek-V3 routing written with masks and torch.topk (a different
  algorithm text) on rows without ties, a pure-Python loop over sorted lists on tiny inputs with ties, one group =
  plain top-k of score + bias, and the fixed answer when every score is -inf (tests/test_oracle_routing.py).
* silu_and_mul_ref -- pinned by a float64 evaluation (at most one rounding step of the
  output type apart), by torch.sigmoid (a different formula), and by the special
  cases silu(0) = 0, silu(g) = g for large g, silu(g) = -0 for very negative g and
  silu(g) - silu(-g) = g.
* rms_norm_ref, fused_add_rms_norm_ref, row_sum_of_squares_f32 -- pinned by a float64
  evaluation (one or two rounding steps of the output type apart), by
  torch.nn.functional.rms_norm on fp32 inputs, by rows of small integers (whose sum of
  squares is exact in any order, so a dropped or repeated element shows), by rows of
  one repeated value (closed form), and by the exact invariance under scaling x by a
  power of two with eps = 0.
* scaled_mm_ref, scaled_mm_ref_postscale -- pinned against each other, a float64
  loop, and the unit-scale/zero-bias closed form.

No function here is "parity unpinned".
"""
from __future__ import annotations

import math
from typing import List, Optional, Tuple

import torch

FP8_DTYPE = torch.float8_e4m3fn
FP8_MAX = 448.0


# --------------------------------------------------------------------------------------
# Activation quantizers
# --------------------------------------------------------------------------------------
def act_quant_ref(
    x: torch.Tensor, block_size: int = 128, scale_fmt: Optional[str] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Restates ``torch_act_quant`` (reference tests/test_act_quant.py:48-98).

    fp32 amax per ``block_size`` group, floor 1e-4, scale = amax * fp32(1/448);
    with ``scale_fmt`` set the scale is rounded up to a power of two by the
    exponent/mantissa bit test of tests/test_act_quant.py:73-85; codes =
    clamp(x * (1/scale), +-448) cast to e4m3fn (round-to-nearest-even).
    """
    assert x.is_contiguous(), "Input tensor must be contiguous"
    assert x.size(-1) % block_size == 0, "Last dim must be divisible by block_size"
    fp8_max_inv = 1.0 / 448.0
    n = x.size(-1)
    x_2d = x.view(-1, n)
    m = x_2d.size(0)
    n_blocks = n // block_size
    xb = x_2d.view(m, n_blocks, block_size).float()
    amax = xb.abs().amax(dim=-1)
    amax = torch.clamp(amax, min=1e-4)
    if scale_fmt is not None:
        scale_raw = amax * fp8_max_inv
        bits = scale_raw.view(torch.int32)
        exp_x = (bits >> 23) & 0xFF
        man = bits & ((1 << 23) - 1)
        log2_ceil = (exp_x - 127 + (man != 0).int()).int()
        scale = ((log2_ceil + 127) << 23).view(torch.float32)
    else:
        scale = amax * fp8_max_inv
    yb = xb * (1.0 / scale.unsqueeze(-1))
    yb = torch.clamp(yb, -FP8_MAX, FP8_MAX)
    y = yb.view(m, n).to(FP8_DTYPE).view(x.shape)
    s = scale.to(torch.float32).view(*x.shape[:-1], n_blocks)
    return y, s


def per_token_group_quant_fp8_ref(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    dtype: torch.dtype = FP8_DTYPE,
    scale_ue8m0: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Restates ``native_per_token_group_quant_fp8``
    (reference tests/test_per_token_group_quant_fp8.py:23-48).

    abs/max/clamp(eps) are done in x's own dtype, then widened to fp32;
    scale = amax * fp32(1/448); optional exp2(ceil(log2(max(|s|,1e-10))));
    codes = clamp(x / scale, +-448) with a true fp32 division.
    """
    assert x.shape[-1] % group_size == 0
    assert x.is_contiguous(), "`x` is not contiguous"
    finfo = torch.finfo(dtype)
    x_ = x.reshape(x.numel() // group_size, group_size)
    amax = x_.abs().max(dim=-1, keepdim=True)[0].clamp(min=eps).to(torch.float32)
    x_s = amax * torch.tensor(1.0 / finfo.max, dtype=torch.float32)
    if scale_ue8m0:
        min_val = torch.tensor(1e-10, dtype=x_s.dtype)
        x_s = torch.exp2(torch.ceil(torch.log2(torch.maximum(x_s.abs(), min_val))))
    x_q = (x_ / x_s).clamp(min=finfo.min, max=finfo.max).to(dtype)
    x_q = x_q.reshape(x.shape)
    x_s = x_s.reshape(x.shape[:-1] + (x.shape[-1] // group_size,))
    return x_q, x_s


def per_token_group_quant_fp8_div_ref(
    x: torch.Tensor, group_size: int, eps: float = 1e-10, dtype: torch.dtype = FP8_DTYPE
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Restates ``torch_per_token_group_quant_fp8``
    (reference tests/test_fused_experts_impl.py:582-601): as above but the scale
    is the true quotient amax / 448 (the form the reference's device kernel and
    its MoE fallback use, src/flag_gems/fused/fused_moe.py:664-668)."""
    assert x.shape[-1] % group_size == 0
    assert x.is_contiguous()
    finfo = torch.finfo(dtype)
    xr = x.reshape(x.numel() // group_size, group_size)
    amax = xr.abs().max(dim=-1, keepdim=True)[0].clamp(min=eps).to(torch.float32)
    x_scales = amax / finfo.max
    x_quant = (xr / x_scales).clamp(min=finfo.min, max=finfo.max).to(dtype)
    x_quant = x_quant.reshape(x.shape)
    x_scales = x_scales.reshape(x.shape[:-1] + (x.shape[-1] // group_size,))
    return x_quant, x_scales


def per_token_group_quant_fp8_kernel_ref(
    x: torch.Tensor, group_size: int, eps: float = 1e-10, dtype: torch.dtype = FP8_DTYPE, scale_ue8m0: bool = False
) -> Tuple[torch.Tensor, torch.Tensor]:
    """The arithmetic of the reference's DEVICE kernel ``_per_token_group_quant_fp8``
    (src/flag_gems/ops/per_token_group_quant_fp8.py:55-70), which its torch test helper does not follow to the bit:
    the group is widened to fp32 first, the floor ``eps`` is an fp32 value (not rounded to the input's dtype), the
    scale is the true quotient ``max(amax, eps) / fp8_max``, optionally ``exp2(ceil(log2(max(|scale|, 1e-10))))``, and the codes
    are ``clamp(y / scale, fp8_min, fp8_max)`` with a true division."""
    assert x.shape[-1] % group_size == 0
    finfo = torch.finfo(dtype)
    y = x.reshape(x.numel() // group_size, group_size).to(torch.float32)
    amax = torch.maximum(y.abs().max(dim=-1, keepdim=True)[0], torch.tensor(eps, dtype=torch.float32))
    y_s = amax / finfo.max
    if scale_ue8m0:
        y_s = torch.exp2(torch.ceil(torch.log2(torch.maximum(y_s.abs(), torch.tensor(1e-10, dtype=torch.float32)))))
    y_q = (y / y_s).clamp(min=finfo.min, max=finfo.max).to(dtype)
    return y_q.reshape(x.shape), y_s.reshape(x.shape[:-1] + (x.shape[-1] // group_size,))


def inv_rope_ref(o: torch.Tensor, positions: torch.Tensor, cos_sin_cache: torch.Tensor, nope_dim: int, rope_dim: int,
                 round_rotated: bool = True) -> torch.Tensor:
    """Restates ``_reference_inv_rope`` (reference tests/test_fused_inv_rope_fp8_quant.py:104-121): the last
    ``rope_dim`` values of every head rotated back by the token's position, pairs interleaved (GPT-J style), in fp32:
    ``x * cos + rotate(x) * (-sin)`` with ``rotate((a, b)) = (-b, a)``.  With ``round_rotated`` the rotated values are
    rounded to ``o``'s dtype (the test helper); without, the result is fp32 and the rotated tail keeps its fp32
    values (what the reference's device kernel quantizes, src/flag_gems/fused/fused_inv_rope_fp8_quant.py:96-113)."""
    half = rope_dim // 2
    cos_sin = cos_sin_cache.index_select(0, positions)
    cos = cos_sin[:, :half].repeat_interleave(2, dim=-1).unsqueeze(1)
    sin = -cos_sin[:, half:].repeat_interleave(2, dim=-1).unsqueeze(1)
    o_pass = o[..., :nope_dim]
    rot = o[..., nope_dim:].float()
    x1, x2 = rot[..., ::2], rot[..., 1::2]
    rotated_half = torch.stack((-x2, x1), dim=-1).flatten(-2)
    rot = rot * cos + rotated_half * sin
    if round_rotated:
        return torch.cat((o_pass, rot.to(o.dtype)), dim=-1)
    return torch.cat((o_pass.float(), rot), dim=-1)


def fused_inv_rope_fp8_quant_ref(
    o: torch.Tensor, positions: torch.Tensor, cos_sin_cache: torch.Tensor, n_groups: int, heads_per_group: int,
    nope_dim: int = 448, rope_dim: int = 64, quant_group_size: int = 128, eps: float = 1e-10,
    tma_aligned_scales: bool = False, round_rotated: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Restates ``native_fused_inv_rope_fp8_quant`` (reference tests/test_fused_inv_rope_fp8_quant.py:124-177):
    inverse RoPE, then per group of ``quant_group_size`` values in fp32: amax floored at ``eps``,
    scale = amax * fp32(1/448), optionally exp2(ceil(log2(max(scale, eps)))), codes = clamp(x / scale, +-448) cast
    to e4m3fn.  Returns (codes [T, G, hpg * head_dim], scales [T, G, blocks] fp32 -- or, with ``tma_aligned_scales``,
    int32 [T, G, hpg] holding the exponent fields of a head's scales, group c in byte c, as ``_pack_ue8m0_scales``,
    :55-64, packs them).

    ``round_rotated=True`` is the test helper to the letter (it rounds the rotated tail to ``o``'s dtype before
    quantizing); the default ``False`` is the reference's device kernel, which quantizes the fp32 values
    (src/flag_gems/fused/fused_inv_rope_fp8_quant.py:96-128) -- the two differ by that one rounding, which is why
    the reference's own test compares them by cosine similarity."""
    o_rot = inv_rope_ref(o, positions, cos_sin_cache, nope_dim, rope_dim, round_rotated)
    num_tokens, _, head_dim = o_rot.shape
    d = heads_per_group * head_dim
    chunks_per_head = head_dim // quant_group_size
    blocks = d // quant_group_size
    o_blocks = o_rot.reshape(num_tokens, n_groups, d).float().reshape(num_tokens, n_groups, blocks, quant_group_size)
    absmax = o_blocks.abs().amax(dim=-1).clamp(min=eps)
    scales = absmax * (1.0 / FP8_MAX)
    if tma_aligned_scales:
        scales = torch.exp2(torch.ceil(torch.log2(scales.clamp(min=eps))))
    codes = (o_blocks / scales.unsqueeze(-1)).clamp(-FP8_MAX, FP8_MAX).to(FP8_DTYPE).reshape(num_tokens, n_groups, d)
    if not tma_aligned_scales:
        return codes, scales
    exps = (scales.reshape(num_tokens, n_groups, heads_per_group, chunks_per_head).contiguous().view(torch.int32) >> 23) & 0xFF
    packed = torch.zeros(exps.shape[:-1], dtype=torch.int32)
    for c in range(chunks_per_head):
        packed |= exps[..., c] << (8 * c)
    return codes, packed


def silu_and_mul_ref(x: torch.Tensor) -> torch.Tensor:
    """``silu(x[..., :d]) * x[..., d:]`` the way the reference's activation kernel computes it
    (src/flag_gems/fused/silu_and_mul.py:13-18, src/flag_gems/fused/fused_moe.py:795-800): the gate in
    fp32, ``g / (1 + exp(-g))``, times the up value, one rounding to the input's dtype.  (The torch
    expression of the reference's MoE check, tests/test_fused_experts_impl.py:629-633, rounds the
    activation and the product separately in bf16; the kernel, restated here, rounds once.)"""
    d = x.shape[-1] // 2
    g = x[..., :d].to(torch.float32)
    u = x[..., d:].to(torch.float32)
    return (g / (1.0 + torch.exp(-g)) * u).to(x.dtype)


def row_sum_of_squares_f32(t: torch.Tensor) -> torch.Tensor:
    """Sum of squares of every row of a float32 [rows, cols] tensor (cols a multiple of 8) in fp32, every
    multiply and add rounded on its own, in the order the HIP library documents for its RMSNorm kernel
    (the reference leaves the order to its compiler, src/flag_gems/ops/rms_norm.py:64): 256 accumulators
    take the 8-element chunks t, t + 256, ... of the row element by element; accumulators 64 k .. 64 k + 63
    are folded with a butterfly at distances 1, 2, 4, 8, 16, 32; the four results are added in order."""
    assert t.dtype == torch.float32 and t.dim() == 2 and t.shape[1] % 8 == 0
    rows, cols = t.shape
    per = -(-(cols // 8) // 256)
    padded = torch.zeros((rows, per * 2048), dtype=torch.float32)
    padded[:, :cols] = t
    v = padded.view(rows, per, 256, 8)
    acc = torch.zeros((rows, 256), dtype=torch.float32)
    for i in range(per):
        for e in range(8):
            sq = v[:, i, :, e] * v[:, i, :, e]
            acc = acc + sq
    acc = acc.view(rows, 4, 64)
    lanes = torch.arange(64)
    for mask in (1, 2, 4, 8, 16, 32):
        acc = acc + acc[:, :, lanes ^ mask]
    w = acc[:, :, 0]
    return ((w[:, 0] + w[:, 1]) + w[:, 2]) + w[:, 3]


def _inverse_rms(t: torch.Tensor, eps: float) -> torch.Tensor:
    """``1 / sqrt(sum / N + eps)`` with every operation correctly rounded to fp32.  Division, square root and
    reciprocal go through float64 and are rounded once more (for these three operations on fp32 operands that
    second rounding cannot change the result: 53 >= 2 * 24 + 2 bits): the vectorised fp32 reciprocal of some
    hosts is an approximation, one or two steps off, which would make this oracle depend on the machine."""
    var = (row_sum_of_squares_f32(t).double() / float(t.shape[1])).float()
    shifted = var + torch.tensor(eps, dtype=torch.float32)
    root = torch.sqrt(shifted.double()).float()
    return (1.0 / root.double()).float()


def rms_norm_ref(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """RMSNorm over the last dimension of a 2-D x as the reference's kernel computes it
    (src/flag_gems/ops/rms_norm.py:54-66): fp32 throughout, ``var = sum(x^2) / N``,
    ``rrms = 1 / sqrt(var + eps)``, the normalised value rounded to x's dtype *before* the multiplication
    by the weight, the product rounded again."""
    xf = x.to(torch.float32)
    x_normed = (xf * _inverse_rms(xf, eps)[:, None]).to(x.dtype)
    return (x_normed.to(torch.float32) * weight.to(torch.float32)).to(x.dtype)


def fused_add_rms_norm_ref(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Residual add + RMSNorm as the reference's looped kernel computes it
    (src/flag_gems/fused/fused_add_rms_norm.py:92-118; the reference uses it for rows over 4096 elements, and its
    single-pass kernel for shorter rows, lines 42-56, rounds differently): ``t = x + residual`` in fp32, the
    new residual is t rounded to the dtype, the variance is ``sum(t^2) / N`` of the *unrounded* t, the
    second pass reads the rounded t back: ``y = T(t) * rrms * w`` rounded once.
    Returns (y, new_residual); the reference writes them over x and residual."""
    t = x.to(torch.float32) + residual.to(torch.float32)
    stored = t.to(x.dtype)
    y = ((stored.to(torch.float32) * _inverse_rms(t, eps)[:, None]) * weight.to(torch.float32)).to(x.dtype)
    return y, stored


# --------------------------------------------------------------------------------------
# DeepGEMM-style casts used to prepare weights (128x128 blocks) and activations
# --------------------------------------------------------------------------------------
def _ceil_to_ue8m0(x: torch.Tensor) -> torch.Tensor:
    """reference tests/test_fp8_einsum.py:63-67."""
    bits = x.abs().float().view(torch.int32)
    exp = ((bits >> 23) & 0xFF) + (bits & 0x7FFFFF).bool().int()
    return (exp.clamp(1, 254) << 23).view(torch.float32)


def per_token_cast_to_fp8_ref(
    x: torch.Tensor, use_ue8m0: bool = False, gran_k: int = 128
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Restates ``per_token_cast_to_fp8`` (reference tests/test_fp8_einsum.py:70-86)."""
    assert x.dim() == 2
    m, n = x.shape
    padded_n = math.ceil(n / gran_k) * gran_k
    x_padded = torch.zeros((m, padded_n), dtype=x.dtype)
    x_padded[:, :n] = x
    x_view = x_padded.view(m, padded_n // gran_k, gran_k)
    x_amax = x_view.abs().float().amax(dim=2).view(m, padded_n // gran_k).clamp(1e-4)
    sf = x_amax / 448.0
    sf = _ceil_to_ue8m0(sf) if use_ue8m0 else sf
    x_fp8 = (
        (x_view * (1.0 / sf.unsqueeze(2)))
        .to(FP8_DTYPE)
        .view(m, padded_n)[:, :n]
        .contiguous()
    )
    return x_fp8, sf


def per_block_cast_to_fp8_ref(
    x: torch.Tensor, use_ue8m0: bool = False, gran_k: int = 128
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Restates ``per_block_cast_to_fp8`` (reference tests/test_fp8_einsum.py:89-103):
    zero-pad to multiples of 128, amax over each (128,128) block in fp32, floor 1e-4,
    sf = amax / 448, codes = x * (1/sf) cast to e4m3fn (no clamp)."""
    assert x.dim() == 2
    m, n = x.shape
    padded_m = math.ceil(m / gran_k) * gran_k
    padded_n = math.ceil(n / gran_k) * gran_k
    x_padded = torch.zeros((padded_m, padded_n), dtype=x.dtype)
    x_padded[:m, :n] = x
    x_view = x_padded.view(-1, gran_k, x_padded.size(1) // gran_k, gran_k)
    x_amax = x_view.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    sf = x_amax / 448.0
    sf = _ceil_to_ue8m0(sf) if use_ue8m0 else sf
    x_scaled = (x_view * (1.0 / sf)).to(FP8_DTYPE)
    return (
        x_scaled.view_as(x_padded)[:m, :n].contiguous(),
        sf.view(x_view.size(0), x_view.size(2)),
    )


# --------------------------------------------------------------------------------------
# Block-scaled GEMM
# --------------------------------------------------------------------------------------
def block_fp8_matmul_dequant_ref(
    A: torch.Tensor,
    B: torch.Tensor,
    As: torch.Tensor,
    Bs: torch.Tensor,
    block_size: List[int],
    output_dtype: torch.dtype = torch.float32,
    compute_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Restates the reference check of tests/test_w8a8_block_fp8_matmul.py:76-100:
    dequantise A per (row, K-block) and B per (N-block, K-block) in fp32, then one
    ``matmul(A_scaled, B_scaled.T)``.  ``compute_dtype=float64`` gives the
    reference's ``--ref cpu`` mode (tests/accuracy_utils.py:287-302)."""
    block_n, block_k = block_size
    k = A.shape[-1]
    n = B.shape[0]
    a2 = A.reshape(-1, k).to(torch.float32)
    as2 = As.reshape(a2.shape[0], -1).to(torch.float32)
    b2 = B.to(torch.float32)
    bs2 = Bs.to(torch.float32)
    num_k_groups = (k + block_k - 1) // block_k
    num_n_groups = (n + block_n - 1) // block_n
    a_scaled = torch.zeros_like(a2)
    for kg in range(num_k_groups):
        ks, ke = kg * block_k, min((kg + 1) * block_k, k)
        a_scaled[:, ks:ke] = a2[:, ks:ke] * as2[:, kg : kg + 1]
    b_scaled = torch.zeros_like(b2)
    for ng in range(num_n_groups):
        ns, ne = ng * block_n, min((ng + 1) * block_n, n)
        for kg in range(num_k_groups):
            ks, ke = kg * block_k, min((kg + 1) * block_k, k)
            b_scaled[ns:ne, ks:ke] = b2[ns:ne, ks:ke] * bs2[ng, kg]
    out = torch.matmul(a_scaled.to(compute_dtype), b_scaled.to(compute_dtype).T)
    return out.reshape(A.shape[:-1] + (n,)).to(output_dtype)


def block_fp8_matmul_tiled_ref(
    a: torch.Tensor,
    b: torch.Tensor,
    a_scales: torch.Tensor,
    b_scales: torch.Tensor,
    block_size: List[int],
    output_dtype: torch.dtype = torch.float32,
    compute_type: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Restates ``torch_w8a8_block_matmul`` (reference
    tests/test_fused_experts_impl.py:531-579): per (K-tile, N-tile) unscaled
    ``matmul`` accumulated into C after multiplying by a_scale[:,kt]*b_scale[nt,kt].
    This is the order of operations of the device kernel
    (src/flag_gems/ops/w8a8_block_fp8_matmul.py:99-109)."""
    a = a.to(compute_type)
    b = b.to(compute_type)
    assert a.shape[-1] == b.shape[-1]
    assert b.ndim == 2 and b_scales.ndim == 2
    block_n, block_k = block_size
    assert (a.shape[-1] + block_k - 1) // block_k == a_scales.shape[-1]
    assert a.shape[:-1] == a_scales.shape[:-1]
    m = a.numel() // a.shape[-1]
    n, k = b.shape
    origin_c_shape = a.shape[:-1] + (n,)
    a = a.reshape(m, a.shape[-1])
    a_scales = a_scales.reshape(m, a_scales.shape[-1]).to(compute_type)
    b_scales = b_scales.to(compute_type)
    n_tiles = (n + block_n - 1) // block_n
    k_tiles = (k + block_k - 1) // block_k
    assert n_tiles == b_scales.shape[0] and k_tiles == b_scales.shape[1]
    c = torch.zeros((m, n), dtype=compute_type)
    for i in range(k_tiles):
        a_t = a[:, i * block_k : min((i + 1) * block_k, k)]
        for j in range(n_tiles):
            b_t = b[j * block_n : min((j + 1) * block_n, n), i * block_k : min((i + 1) * block_k, k)]
            scale = a_scales[:, i : i + 1] * b_scales[j][i]
            c[:, j * block_n : min((j + 1) * block_n, n)] += torch.matmul(a_t, b_t.t()) * scale
    return c.reshape(origin_c_shape).to(output_dtype)


def grouped_block_fp8_matmul_ref(
    a: torch.Tensor,
    b: torch.Tensor,
    a_scales: torch.Tensor,
    b_scales: torch.Tensor,
    offs: torch.Tensor,
    block_size: List[int],
    output_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Rows ``offs[e-1]:offs[e]`` of ``a`` [M, K] times weight matrix ``b[e]`` [N, K] with
    scales ``b_scales[e]``: the per-expert loop of the reference's block-fp8 MoE check
    (tests/test_fused_experts_impl.py:636-646, each expert's rows through
    ``torch_w8a8_block_matmul``) over rows already sorted by expert, the segments given as
    the cumulative int32 ends of ``aten::_scaled_grouped_mm``
    (src/flag_gems/ops/scaled_grouped_mm.py:111-114, 275-287).  Rows at or past the last end
    come back as zeros (the device leaves them unwritten)."""
    m = a.shape[0]
    e_count, n, _ = b.shape
    assert offs.numel() == e_count
    c = torch.zeros((m, n), dtype=output_dtype)
    begin = 0
    for e in range(e_count):
        end = int(offs[e])
        if end > begin:
            c[begin:end] = block_fp8_matmul_tiled_ref(
                a[begin:end], b[e], a_scales[begin:end], b_scales[e], block_size, output_dtype
            )
        begin = max(begin, end)
    return c


def block_fp8_moe_ref(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    w1_scale: torch.Tensor,
    w2_scale: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    block_shape: List[int],
    expert_map: Optional[torch.Tensor] = None,
    tokens: Optional[torch.Tensor] = None,
    kernel_activation: bool = True,
) -> torch.Tensor:
    """Restates ``torch_w8a8_block_fp8_moe`` (reference tests/test_fused_experts_impl.py:604-662): every routed slot
    (token t, choice j) goes through quantize (``amax / 448``) -> ``torch_w8a8_block_matmul`` with W1 of its expert
    -> SiLU-and-mul -> quantize -> ``torch_w8a8_block_matmul`` with W2, each GEMM rounded to the activations' dtype,
    and the slot results are weighted and summed per token in that dtype.

    ``expert_map`` (global expert -> local expert or -1): slots of experts that are not local contribute zeros, as
    the reference's kernel writes them (src/flag_gems/fused/fused_moe.py:1114, 2128-2129).  ``tokens``: evaluate
    only these token rows (the full-size configurations are checked on a sample).  ``kernel_activation``: the
    activation rounds once (``silu_and_mul_ref``, what the reference's kernel does) instead of twice in the
    activations' dtype (the torch expression at :629-633); both are within the test's tolerance of each other.
    The weighted sum follows the reference's expression: slot result times weight rounded to the dtype, summed over
    the choices by torch in that dtype."""
    if tokens is not None:
        hidden_states, topk_weights, topk_ids = hidden_states[tokens], topk_weights[tokens], topk_ids[tokens]
    batch, hidden = hidden_states.shape
    topk = topk_ids.size(1)
    _, block_k = block_shape
    expanded = hidden_states.view(batch, -1, hidden).repeat(1, topk, 1).reshape(-1, hidden)
    out = torch.zeros(batch * topk, w2.shape[1], dtype=hidden_states.dtype)
    flat_ids = topk_ids.reshape(-1).to(torch.int64)
    if expert_map is not None:
        flat_ids = expert_map.to(torch.int64)[flat_ids]
    hq, hs = per_token_group_quant_fp8_div_ref(expanded.contiguous(), block_k)

    def activation(x):
        if kernel_activation:
            return silu_and_mul_ref(x)
        d = x.shape[-1] // 2
        return torch.nn.functional.silu(x[..., :d]) * x[..., d:]

    for e in range(w1.shape[0]):
        mask = flat_ids == e
        if mask.sum():
            inter = block_fp8_matmul_tiled_ref(hq[mask], w1[e], hs[mask], w1_scale[e], block_shape, hidden_states.dtype)
            aq, a_s = per_token_group_quant_fp8_div_ref(activation(inter).contiguous(), block_k)
            out[mask] = block_fp8_matmul_tiled_ref(aq, w2[e], a_s, w2_scale[e], block_shape, hidden_states.dtype)
    return (out.view(batch, -1, w2.shape[1]) * topk_weights.reshape(batch, -1, 1).to(out.dtype)).sum(dim=1)


def fp8_block_einsum_ref(
    x_data: torch.Tensor,
    x_scale: torch.Tensor,
    y_data: torch.Tensor,
    y_scale: torch.Tensor,
    block_shape: List[int],
) -> torch.Tensor:
    """Restates ``torch_fp8_block_einsum_reference`` (reference tests/test_fp8_einsum.py:130-160):
    x [b, h, r] dequantised per (token, head, K-block), y [h, d, r] per (head, N-block, K-block), then
    ``einsum("bhr,hdr->bhd")`` in fp32."""
    block_n, block_k = block_shape
    b, h, r = x_data.shape
    d = y_data.shape[1]
    x_f = x_data.to(torch.float32)
    y_f = y_data.to(torch.float32)
    x_deq = torch.empty_like(x_f)
    for kt in range(x_scale.shape[-1]):
        ks, ke = kt * block_k, min((kt + 1) * block_k, r)
        x_deq[:, :, ks:ke] = x_f[:, :, ks:ke] * x_scale[:, :, kt : kt + 1]
    y_deq = torch.empty_like(y_f)
    for nt in range(y_scale.shape[1]):
        ns, ne = nt * block_n, min((nt + 1) * block_n, d)
        for kt in range(x_scale.shape[-1]):
            ks, ke = kt * block_k, min((kt + 1) * block_k, r)
            y_deq[:, ns:ne, ks:ke] = y_f[:, ns:ne, ks:ke] * y_scale[:, nt, kt].view(h, 1, 1)
    return torch.einsum("bhr,hdr->bhd", x_deq, y_deq)


def make_fp8_einsum_inputs(b: int, h: int, r: int, d: int, seed: int = 0):
    """Inputs as the reference test builds them (tests/test_fp8_einsum.py:105-127): x, y ~ N(0,1) bf16,
    x cast per token (1 x 128, power-of-two scales), y per head per 128 x 128 block (power-of-two scales)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((b, h, r), generator=g).bfloat16()
    y = torch.randn((h, d, r), generator=g).bfloat16()
    xq, xs = per_token_cast_to_fp8_ref(x.view(-1, r), use_ue8m0=True)
    yq = torch.empty((h, d, r), dtype=FP8_DTYPE)
    ys = torch.empty((h, (d + 127) // 128, (r + 127) // 128), dtype=torch.float32)
    for i in range(h):
        yq[i], ys[i] = per_block_cast_to_fp8_ref(y[i], use_ue8m0=True)
    return xq.view(b, h, r), xs.view(b, h, -1), yq, ys


def topk_softmax_ref(gating: torch.Tensor, topk: int, renormalize: bool = False):
    """Restates the reference's routing kernel ``topk_gating_softmax_kernel``
    (src/flag_gems/fused/topk_softmax.py:44-82; its own test compares with vLLM's CUDA operator, which is not in
    this image): fp32 probabilities exp(x - max) / (sum + 1e-8), then ``topk`` rounds of (largest remaining value,
    first index that holds it), the taken entry set to -inf; with ``renormalize`` the selected values are divided by
    (their running sum + 1e-8).  Returns (weights fp32 [T, k], indices int64 [T, k], token_expert_indices int32
    [T, k] = k * T + t)."""
    x = gating.float()
    tokens = x.shape[0]
    e = torch.exp(x - x.max(dim=1, keepdim=True).values)
    probs = e / (e.sum(dim=1, keepdim=True) + 1e-8)
    weights = torch.empty(tokens, topk, dtype=torch.float32)
    indices = torch.empty(tokens, topk, dtype=torch.int64)
    selected_sum = torch.zeros(tokens, dtype=torch.float32)
    for ki in range(topk):
        cur, arg = torch.max(probs, dim=1)          # the first maximal value's index
        weights[:, ki], indices[:, ki] = cur, arg
        selected_sum = selected_sum + cur
        probs = probs.scatter(1, arg.unsqueeze(1), float("-inf"))
    if renormalize:
        weights = weights / (selected_sum + 1e-8).unsqueeze(1)
    source = (torch.arange(topk, dtype=torch.int32).unsqueeze(0) * tokens + torch.arange(tokens, dtype=torch.int32).unsqueeze(1))
    return weights, indices, source


def grouped_topk_ref(scores: torch.Tensor, n_group: int, topk_group: int, topk: int, renormalize: bool,
                     routed_scaling_factor: float, bias: torch.Tensor, scoring_func: int = 0):
    """Restates the reference's group-limited routing (src/flag_gems/fused/grouped_topk.py:256-355 with its kernels
    ``topk_with_k2_triton`` :25-78 and ``group_idx_and_topk_triton`` :81-253; its own test compares with vLLM's CUDA
    operator, which is not in this image).  All sums of 16-bit tensors are rounded to their type as the kernels'
    loads and stores round them: s = scores or sigmoid(scores) in the scores' type, sb = s + bias, group score = the
    two largest sb of the group added (rounded), not-finite group scores = -inf, the ``topk_group`` largest groups
    (ties: lower group), ``topk`` rounds of (largest remaining sb among their experts, first index), weights = s of
    the selected * factor, over (their sum + 1e-20) with ``renormalize``; experts 0 .. topk-1 at 1 / topk each when no
    group score is above -inf.  Returns (fp32 [T, topk], int32 [T, topk])."""
    tokens, experts = scores.shape
    per = experts // n_group
    bias = bias.to(scores.dtype).flatten()
    s = torch.sigmoid(scores.float()).to(scores.dtype) if scoring_func == 1 else scores
    sb = s + bias
    grouped = sb.float().view(tokens, n_group, per)
    max1 = grouped.max(dim=-1).values
    if per >= 2:
        max2 = grouped.topk(2, dim=-1).values[..., 1]
    else:
        max2 = torch.full_like(max1, float("-inf"))
    gs = (max1 + max2).to(scores.dtype).float()
    gs = torch.where(torch.isfinite(gs) | (gs == float("-inf")), gs, torch.full_like(gs, float("-inf")))
    proceed = gs.max(dim=1).values != float("-inf")
    order = torch.sort(gs, dim=1, descending=True, stable=True).indices[:, : min(topk_group, n_group)]
    chosen = torch.zeros(tokens, n_group, dtype=torch.bool).scatter(1, order, True)
    sel = torch.where(chosen.repeat_interleave(per, dim=1), sb.float(), torch.full((tokens, experts), float("-inf")))
    values = torch.empty(tokens, topk, dtype=torch.float32)
    ids = torch.empty(tokens, topk, dtype=torch.int64)
    for ki in range(topk):
        arg = torch.max(sel, dim=1).indices
        ids[:, ki] = arg
        values[:, ki] = s.float().gather(1, arg.unsqueeze(1)).squeeze(1)
        sel = sel.scatter(1, arg.unsqueeze(1), float("-inf"))
    if renormalize:
        total = torch.zeros(tokens, dtype=torch.float32)
        for ki in range(topk):
            total = total + values[:, ki]
        scale = torch.tensor(routed_scaling_factor, dtype=torch.float32) / (total + 1e-20)
        values = values * scale.unsqueeze(1)
    else:
        values = values * torch.tensor(routed_scaling_factor, dtype=torch.float32)
    values = torch.where(proceed.unsqueeze(1), values, torch.full_like(values, 1.0 / topk))
    ids = torch.where(proceed.unsqueeze(1), ids, torch.arange(topk).expand(tokens, topk))
    return values, ids.to(torch.int32)


def make_moe_rows(tokens: int, experts: int = 8, top_k: int = 2, seed: int = 0) -> torch.Tensor:
    """Cumulative int32 row ends of ``tokens * top_k`` rows sorted by expert, with expert loads
    proportional to a Zipf(1.1) law over a seeded permutation of the experts (the synthetic
    routing of the Mixtral-shaped benchmark configuration; no counterpart in the reference)."""
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(experts, generator=g)
    p = torch.zeros(experts, dtype=torch.float64)
    p[perm] = 1.0 / torch.arange(1, experts + 1, dtype=torch.float64) ** 1.1
    p /= p.sum()
    ids = torch.multinomial(p, tokens * top_k, replacement=True, generator=g)
    counts = torch.bincount(ids, minlength=experts)
    return torch.cumsum(counts, 0).to(torch.int32)


# --------------------------------------------------------------------------------------
# Per-tensor / per-token x per-channel scaled GEMM
# --------------------------------------------------------------------------------------
def scaled_mm_ref(
    a: torch.Tensor,
    b: torch.Tensor,
    scale_a: torch.Tensor,
    scale_b: torch.Tensor,
    out_dtype: torch.dtype,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Restates ``baseline_scaled_mm`` (reference tests/test_cutlass_scaled_mm.py:154-187)
    for scalar / per-row ``scale_a`` ([M,1] or [1]) and scalar / per-column ``scale_b``
    ([1,N] or [1]): scale the operands in fp32, one fp32 ``mm``, cast to ``out_dtype``,
    then add the bias in ``out_dtype``."""
    sa = scale_a.reshape(-1, 1) if scale_a.numel() > 1 else scale_a.reshape(1, 1)
    sb = scale_b.reshape(1, -1) if scale_b.numel() > 1 else scale_b.reshape(1, 1)
    lhs = sa * a.to(torch.float32)
    rhs = sb * b.to(torch.float32)
    output = torch.mm(lhs, rhs).to(out_dtype)
    if bias is not None:
        output = output + bias
    return output


def scaled_mm_ref_postscale(
    mat1: torch.Tensor,
    mat2: torch.Tensor,
    scale_a: torch.Tensor,
    scale_b: torch.Tensor,
    bias: Optional[torch.Tensor],
    out_dtype: Optional[torch.dtype],
    compute_dtype: torch.dtype = torch.float64,
) -> torch.Tensor:
    """Restates ``_reference_scaled_mm`` (reference tests/test_scaled_mm.py:111-124):
    ``mm`` first (in the reference's float64 "to_reference" precision), then the two
    scales, then the bias, one final cast."""
    rows, cols = mat1.shape[0], mat2.shape[1]

    def shaped(scale, is_left):
        if scale.numel() == 1:
            return scale
        if scale.ndim == 1:
            if is_left and scale.shape[0] == rows:
                return scale.reshape(rows, 1)
            if not is_left and scale.shape[0] == cols:
                return scale.reshape(1, cols)
        return scale

    ref = mat1.to(compute_dtype).mm(mat2.to(compute_dtype))
    ref = ref * shaped(scale_a.to(compute_dtype), True)
    ref = ref * shaped(scale_b.to(compute_dtype), False)
    if bias is not None:
        ref = ref + bias.to(compute_dtype)
    return ref.to(out_dtype or mat1.dtype)


# --------------------------------------------------------------------------------------
# Synthetic inputs of the benchmark configurations
# --------------------------------------------------------------------------------------
def make_config1(seed: int = 0):
    """The CPU-runnable benchmark configuration: X bf16 [64,1024] ~N(0,1), W bf16 [512,1024] ~N(0,0.02),
    generator order X then W, one ``torch.manual_seed(seed)``."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(64, 1024, generator=g).bfloat16()
    w = (0.02 * torch.randn(512, 1024, generator=g)).bfloat16()
    return x, w


def run_config1(seed: int = 0):
    """Full CPU reference path of config 1: act_quant -> 128x128 weight quant ->
    block-scaled matmul -> bf16 [64,512]."""
    x, w = make_config1(seed)
    xq, xs = act_quant_ref(x, 128)
    wq, ws = per_block_cast_to_fp8_ref(w, use_ue8m0=False)
    c = block_fp8_matmul_tiled_ref(xq, wq, xs, ws, [128, 128], torch.bfloat16)
    return dict(x=x, w=w, xq=xq, xs=xs, wq=wq, ws=ws, c=c)
