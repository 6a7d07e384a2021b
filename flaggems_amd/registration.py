"""Installs the FP8 quantized-linear operators into PyTorch's dispatcher.

Mirrors the part of the reference's registration layer that concerns this path:
  enable / only_enable / use_gems / all_registered_ops / all_registered_keys
      src/flag_gems/__init__.py:1183-1336, src/flag_gems/runtime/op_registrar.py:116-159
  the two ATen entries ("_scaled_mm", "_scaled_mm.out")   src/flag_gems/__init__.py:230-231
  patch_empty_vllm and the vLLM ``_C`` schemas              src/flag_gems/patches/patch_util.py:59-161,
                                                            src/flag_gems/patches/patch_vllm_all.py:643-717
There is one device (gfx950, dispatch key "CUDA" under PyTorch-ROCm) and one implementation per
operator, so no vendor detection, condition lambdas or tuning tables are involved.
"""
from __future__ import annotations

import logging
import os
import warnings
from typing import Iterable, List, Optional, Tuple

import torch

from .act_quant import per_token_group_fp8_quant_into, silu_and_mul_packed_out
from .cutlass_scaled_mm import cutlass_scaled_mm
from .fused_moe import moe_align_block_size_triton, moe_sum
from .moe_routing import grouped_topk, topk_softmax
from .norm_quant import rms_norm_out
from .scaled_mm import scaled_mm, scaled_mm_out

logger = logging.getLogger("flag_gems")

DISPATCH_KEY = "CUDA"

# (aten overload name, implementation) -- the hot-path subset of the reference's _FULL_CONFIG
_FULL_CONFIG: Tuple[Tuple[str, object], ...] = (
    ("_scaled_mm", scaled_mm),
    ("_scaled_mm.out", scaled_mm_out),
)

aten_lib = torch.library.Library("aten", "IMPL")


class GeneralOpRegistrar:
    """Registers the selected (key, fn) pairs into ``lib`` and remembers what it registered."""

    def __init__(self, config, user_include_ops=None, user_exclude_ops=None, lib=None, **_ignored):
        self.lib = lib
        include = set(user_include_ops or [])
        exclude = set(user_exclude_ops or [])
        self.registered: List[Tuple[str, object]] = []
        for key, fn in config:
            name = fn.__name__
            if include and name not in include and key not in include:
                continue
            if not include and (name in exclude or key in exclude):
                continue
            try:
                lib.impl(key, fn, DISPATCH_KEY)
                self.registered.append((key, fn))
            except Exception as exc:  # same policy as the reference: warn and continue
                warnings.warn(f"flag_gems: registering {key} failed: {exc}")

    def get_all_ops(self):
        return [fn.__name__ for _, fn in self.registered]

    def get_all_keys(self):
        return [key for key, _ in self.registered]


current_work_registrar: Optional[GeneralOpRegistrar] = None


def _as_list(names) -> List[str]:
    if names is None or names == "default":
        return []
    if isinstance(names, str):
        if names.endswith((".yml", ".yaml")):
            import yaml

            with open(names) as f:
                data = yaml.safe_load(f) or []
            if isinstance(data, dict):
                data = data.get("include") or data.get("exclude") or []
            return list(data)
        return [names]
    return list(names)


class _LogOncePerLocation(logging.Filter):
    """Passes the first record of every call site (file, line) and drops the repeats: with ``once=True`` the record
    file lists each operator call site once instead of once per call
    (the reference's LogOncePerLocationFilter, src/flag_gems/logging_utils.py:34-45)."""

    def __init__(self):
        super().__init__()
        self.seen = set()

    def filter(self, record):
        key = (record.pathname, record.lineno)
        if key in self.seen:
            return False
        self.seen.add(key)
        return True


def _setup_logging(record: bool, once: bool, path: Optional[str]) -> None:
    """The reference's setup_flaggems_logging (src/flag_gems/logging_utils.py:60-84): with ``record`` a file handler
    on the ``flag_gems`` logger (a new call replaces the previous one's), the same line format, DEBUG level, no
    propagation; ``once`` filters repeats per call site.  Default file: ~/.flaggems/oplist.log."""
    if not record:
        return
    _teardown_logging()
    filename = os.path.expanduser(path) if path else os.path.join(os.path.expanduser("~"), ".flaggems", "oplist.log")
    parent = os.path.dirname(os.path.abspath(filename))
    os.makedirs(parent, exist_ok=True)
    handler = logging.FileHandler(filename, mode="w")
    handler.setFormatter(logging.Formatter("[%(levelname)s] %(name)s.%(funcName)s: %(message)s"))
    handler.set_name("flag_gems_record")
    if once:
        handler.addFilter(_LogOncePerLocation())
    logger.addHandler(handler)
    logger.setLevel(logging.DEBUG)
    logger.propagate = False


def _teardown_logging() -> None:
    for h in list(logger.handlers):
        if h.get_name() == "flag_gems_record":
            logger.removeHandler(h)
            h.close()


def enable(lib=aten_lib, unused=None, registrar=GeneralOpRegistrar, record=False, once=False, path=None):
    """Register every operator of this build except those named in ``unused``."""
    global current_work_registrar
    current_work_registrar = registrar(_FULL_CONFIG, user_include_ops=[], user_exclude_ops=_as_list(unused), lib=lib)
    _setup_logging(record, once, path)


def only_enable(lib=aten_lib, include=None, registrar=GeneralOpRegistrar, record=False, once=False, path=None):
    """Register only the operators named in ``include`` (function names or ATen keys)."""
    include_ops = _as_list(include)
    if not include_ops:
        warnings.warn("only_enable failed: No include entries resolved from list or yaml.")
        return
    global current_work_registrar
    current_work_registrar = registrar(_FULL_CONFIG, user_include_ops=include_ops, user_exclude_ops=[], lib=lib)
    _setup_logging(record, once, path)


class use_gems:
    """Context manager: operators are registered on entry and removed on exit.
    ``include`` has priority over ``exclude``."""

    def __init__(self, exclude=None, include=None, record=False, once=False, path=None):
        self.lib = torch.library.Library("aten", "IMPL")
        self.exclude = exclude if isinstance(exclude, (list, tuple, set, str)) else []
        self.include = include if isinstance(include, (list, tuple, set, str)) else []
        self.record, self.once, self.path = record, once, path

    def __enter__(self):
        if self.include:
            only_enable(lib=self.lib, include=self.include, record=self.record, once=self.once, path=self.path)
        else:
            enable(lib=self.lib, unused=self.exclude, record=self.record, once=self.once, path=self.path)
        return self

    def __exit__(self, exc_type, exc_val, exc_tb):
        global current_work_registrar
        self.lib._destroy()
        del self.lib
        current_work_registrar = None
        if self.record:
            _teardown_logging()
        return False


def all_registered_ops():
    return current_work_registrar.get_all_ops() if current_work_registrar else []


def all_registered_keys():
    return current_work_registrar.get_all_keys() if current_work_registrar else []


# --------------------------------------------------------------------------------------
# vLLM ``_C`` namespace
# --------------------------------------------------------------------------------------
_VLLM_OPS_SIGNATURES = {
    "cutlass_scaled_mm": "(Tensor(a!) out, Tensor input, Tensor weight, "
    "Tensor scale_a, Tensor scale_b, Tensor? bias=None) -> ()",
    "per_token_group_fp8_quant": "(Tensor input, Tensor(a!) output_q, "
    "Tensor(b!) output_s, int group_size, float eps, float fp8_min, "
    "float fp8_max, bool scale_ue8m0=False) -> ()",
    "rms_norm": "(Tensor(a!) result, Tensor input, Tensor weight, float epsilon) -> ()",
    "silu_and_mul": "(Tensor(a!) out, Tensor input) -> ()",
}


def custom_cutlass_scaled_mm(output, input, weight, scale_a, scale_b, bias=None):
    return cutlass_scaled_mm(output, input, weight, scale_a, scale_b, bias)


def custom_per_token_group_fp8_quant(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0=False):
    per_token_group_fp8_quant_into(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0)


def custom_rms_norm_out(result, input, weight, epsilon):
    rms_norm_out(result, input, list(weight.size()), weight, epsilon)


def custom_silu_and_mul(out, input):
    silu_and_mul_packed_out(out, input)


_VLLM_IMPLS = {
    "cutlass_scaled_mm": custom_cutlass_scaled_mm,
    "per_token_group_fp8_quant": custom_per_token_group_fp8_quant,
    "rms_norm": custom_rms_norm_out,
    "silu_and_mul": custom_silu_and_mul,
}

# the operators of vLLM's ``_moe_C`` namespace that the reference implements: routing, alignment, the sum over the slots
# (src/flag_gems/patches/patch_util.py:74-85, patch_vllm_all.py:306-359, 628-633)
_VLLM_MOE_OPS_SIGNATURES = {
    "moe_align_block_size": "(Tensor topk_ids, int num_experts, "
    "int block_size, Tensor(a!) sorted_token_ids, Tensor(b!) experts_ids, "
    "Tensor(c!) num_tokens_post_pad) -> ()",
    "moe_sum": "(Tensor input, Tensor(a!) output) -> ()",
    "topk_softmax": "(Tensor(a!) topk_weights, Tensor(b!) topk_indices, Tensor(c!) token_expert_indices, "
    "Tensor gating_output, bool renormalize=False) -> ()",
    "grouped_topk": "(Tensor scores, int n_group, int topk_group, int topk, bool renormalize, "
    "float routed_scaling_factor, Tensor bias, int scoring_func=0) -> (Tensor, Tensor)",
}


def custom_moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids, num_tokens_post_pad):
    moe_align_block_size_triton(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids, num_tokens_post_pad)


def custom_moe_sum(input, output):
    moe_sum(input, output)


def custom_topk_softmax(topk_weights, topk_indices, token_expert_indices, gating_output, renormalize=False):
    topk_softmax(topk_weights, topk_indices, token_expert_indices, gating_output, renormalize)


def custom_moe_grouped_topk(gating_output, n_group, topk_group, topk, renormalize, routed_scaling_factor, bias, scoring_func=0):
    return grouped_topk(scores=gating_output, n_group=n_group, topk_group=topk_group, topk=topk, renormalize=renormalize,
                        routed_scaling_factor=routed_scaling_factor, bias=bias, scoring_func=scoring_func)


_VLLM_MOE_IMPLS = {
    "moe_align_block_size": custom_moe_align_block_size,
    "moe_sum": custom_moe_sum,
    "topk_softmax": custom_topk_softmax,
    "grouped_topk": custom_moe_grouped_topk,
}

_vllm_libs: List[torch.library.Library] = []
_vllm_patched = False


def _op_defined(namespace: str, name: str) -> bool:
    try:
        getattr(getattr(torch.ops, namespace), name)
        return True
    except (AttributeError, RuntimeError):
        return False


def patch_empty_vllm(verbose: bool = False) -> None:
    """Define (when vLLM has not) and implement the ``_C`` and ``_moe_C`` operators of this path.  Idempotent."""
    global _vllm_patched
    if _vllm_patched:
        return
    for namespace, signatures, impls in (("_C", _VLLM_OPS_SIGNATURES, _VLLM_IMPLS),
                                        ("_moe_C", _VLLM_MOE_OPS_SIGNATURES, _VLLM_MOE_IMPLS)):
        for name, schema in signatures.items():
            if not _op_defined(namespace, name):
                def_lib = torch.library.Library(namespace, "FRAGMENT")
                def_lib.define(name + schema)
                _vllm_libs.append(def_lib)
            impl_lib = torch.library.Library(namespace, "IMPL")
            impl_lib.impl(name, impls[name], DISPATCH_KEY)
            _vllm_libs.append(impl_lib)
            if verbose:
                logger.info("patched %s::%s", namespace, name)
    _vllm_patched = True


def apply_gems_patches_to_vllm(verbose: bool = False) -> None:
    """Override vLLM's ``_C`` operators of this path with the gfx950 kernels."""
    patch_empty_vllm(verbose)
