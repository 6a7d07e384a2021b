"""flaggems_amd: MI355X (gfx950) implementation of FlagGems' FP8 quantized-linear operators.

The public names, signatures and registration entry points follow the reference package
``flag_gems`` for this path (see each module's docstring for file:line citations); the compute is
hand-written HIP reached through the C ABI in include/flaggems_amd.h.  Importing the package does
not touch a GPU and does not load the shared library; the first operator call does, and fails
loudly if the library has not been built (``python -m flaggems_amd.build``).
"""
from .act_quant import (  # noqa: F401
    SUPPORTED_FP8_DTYPE,
    act_quant_triton,
    get_group_quant_rule,
    per_block_cast_to_fp8,
    per_token_cast_to_fp8,
    per_token_group_quant_fp8,
    set_group_quant_rule,
    silu_and_mul_packed,
    silu_and_mul_packed_out,
    silu_and_mul_per_token_group_quant_fp8,
)
from .cutlass_scaled_mm import SM_VERSION_NUM, cutlass_scaled_mm, get_sm_version_num  # noqa: F401
from .fp8_einsum import fp8_einsum, w8a8_block_fp8_bmm  # noqa: F401
from .fused_inv_rope_fp8_quant import fused_inv_rope_fp8_quant  # noqa: F401
from .fused_moe import (  # noqa: F401
    fused_experts_impl,
    inplace_fused_experts,
    outplace_fused_experts,
    moe_align_block_size,
    moe_align_block_size_triton,
    moe_sort_slots,
    moe_sum,
)
from .grouped_block_fp8_matmul import (  # noqa: F401
    group_ends_from_expert_ids,
    grouped_w8a8_block_fp8_matmul,
    local_rows_from_moe_align,
)
from .moe_routing import grouped_topk, topk_softmax  # noqa: F401
from .norm_quant import fused_add_rms_norm, rms_norm, rms_norm_out, rms_norm_per_token_group_quant_fp8  # noqa: F401
from .registration import (  # noqa: F401
    all_registered_keys,
    all_registered_ops,
    apply_gems_patches_to_vllm,
    enable,
    only_enable,
    patch_empty_vllm,
    use_gems,
)
from .scaled_mm import scaled_mm, scaled_mm_out  # noqa: F401
from .w8a8_block_fp8_matmul import fp8_matmul, fp8_matmul_noop, w8a8_block_fp8_matmul  # noqa: F401

__version__ = "0.1.0"
device = "cuda"  # PyTorch-ROCm device type of an MI355X
vendor_name = "amd"

__all__ = [
    "SUPPORTED_FP8_DTYPE",
    "act_quant_triton",
    "all_registered_keys",
    "all_registered_ops",
    "apply_gems_patches_to_vllm",
    "cutlass_scaled_mm",
    "enable",
    "fp8_einsum",
    "fp8_matmul",
    "fp8_matmul_noop",
    "fused_add_rms_norm",
    "fused_experts_impl",
    "fused_inv_rope_fp8_quant",
    "get_group_quant_rule",
    "grouped_topk",
    "grouped_w8a8_block_fp8_matmul",
    "group_ends_from_expert_ids",
    "local_rows_from_moe_align",
    "moe_sort_slots",
    "inplace_fused_experts",
    "outplace_fused_experts",
    "moe_align_block_size",
    "moe_align_block_size_triton",
    "moe_sum",
    "only_enable",
    "patch_empty_vllm",
    "per_block_cast_to_fp8",
    "per_token_cast_to_fp8",
    "per_token_group_quant_fp8",
    "rms_norm",
    "rms_norm_out",
    "rms_norm_per_token_group_quant_fp8",
    "scaled_mm",
    "scaled_mm_out",
    "set_group_quant_rule",
    "silu_and_mul_packed",
    "silu_and_mul_packed_out",
    "silu_and_mul_per_token_group_quant_fp8",
    "topk_softmax",
    "use_gems",
    "w8a8_block_fp8_bmm",
    "w8a8_block_fp8_matmul",
]
