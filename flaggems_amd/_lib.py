"""ctypes binding of libflaggems_amd.so (the C ABI declared in include/flaggems_amd.h).

The library is the only implementation of the operators: there is no Python, torch or CPU
fallback.  Loading fails loudly when the shared library has not been built.
"""
from __future__ import annotations

import ctypes
import os
import threading
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_uint64, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libflaggems_amd.so")

# enums of include/flaggems_amd.h
FG_OK = 0
FG_ERR_INVALID_ARG, FG_ERR_UNSUPPORTED, FG_ERR_WORKSPACE, FG_ERR_LAUNCH = -1, -2, -3, -4
FG_BF16, FG_F16, FG_F32, FG_FP8_E4M3FN, FG_FP8_E5M2 = 0, 1, 2, 3, 4
FG_SCALE_MUL_INV, FG_SCALE_DIV = 0, 1
FG_QUOT_RECIP_MUL, FG_QUOT_DIV = 0, 1
FG_POW2_NONE, FG_POW2_BITS, FG_POW2_LOG2, FG_POW2_BITS_CLAMPED = 0, 1, 2, 3
FG_WORKSPACE_COUNTER_BYTES = 16384
FG_NOALLOC_SCRATCH_BYTES = 32 << 20

DTYPE_CODE = {
    torch.bfloat16: FG_BF16,
    torch.float16: FG_F16,
    torch.float32: FG_F32,
    torch.float8_e4m3fn: FG_FP8_E4M3FN,
    torch.float8_e5m2: FG_FP8_E5M2,
}

# name -> (restype, argtypes); must list every symbol the header declares
SIGNATURES = {
    "fg_version": (c_int, []),
    "fg_last_error_string": (c_char_p, []),
    "fg_stream_capture_id": (c_uint64, [c_void_p]),
    "fg_stream_read_probe": (c_int, [c_void_p, c_size_t, c_void_p, c_void_p]),
    "fg_mfma_issue_probe": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "fg_group_quant_fp8": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p, c_int64, c_int64,
         c_int64, c_float, c_float, c_float, c_float, c_int, c_int, c_int, c_void_p],
    ),
    "fg_block_quant_fp8": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p, c_int64, c_int64,
         c_int64, c_int64, c_float, c_float, c_float, c_float, c_int, c_int, c_int, c_void_p],
    ),
    "fg_silu_mul_group_quant_fp8": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p, c_int64, c_int64,
         c_int64, c_float, c_float, c_float, c_float, c_int, c_int, c_int, c_void_p],
    ),
    "fg_rms_norm_group_quant_fp8": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_float, c_void_p, c_int64,
         c_void_p, c_int, c_int64, c_void_p, c_int64, c_int64,
         c_int64, c_float, c_float, c_float, c_float, c_int, c_int, c_int, c_void_p],
    ),
    "fg_silu_mul": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p]),
    "fg_act_quant_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p]),
    "fg_block_fp8_gemm": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
         c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p],
    ),
    "fg_block_fp8_gemm_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "fg_block_fp8_gemm_pow2_scales": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
         c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p],
    ),
    "fg_block_fp8_gemm_noalloc": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
         c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p],
    ),
    "fg_batched_block_fp8_gemm": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64,
         c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int,
         c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p],
    ),
    "fg_grouped_block_fp8_gemm": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64,
         c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_int64,
         c_int64, c_int64, c_void_p, c_size_t, c_void_p],
    ),
    "fg_grouped_block_fp8_gemm_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "fg_scaled_fp8_gemm": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
         c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p],
    ),
    "fg_scaled_gemm": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
         c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p],
    ),
    "fg_scaled_int8_gemm": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
         c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p],
    ),
    "fg_scaled_int8_gemm_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "fg_scaled_fp8_gemm_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "fg_batched_block_fp8_gemm_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64]),
}

_lib = None
_lock = threading.Lock()


class FlagGemsAmdError(RuntimeError):
    """A C-ABI call returned a negative status."""


def load() -> ctypes.CDLL:
    """Load the shared library once; raise if it is missing (no fallback exists)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m flaggems_amd.build` "
                "(hipcc --offload-arch=gfx950).  flaggems_amd has no fallback implementation."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    if status == FG_OK:
        return
    msg = load().fg_last_error_string()
    text = msg.decode("utf-8", "replace") if msg else ""
    if status == FG_ERR_UNSUPPORTED:
        raise NotImplementedError(f"{what}: {text}")
    raise FlagGemsAmdError(f"{what} failed with status {status}: {text}")


def require_gpu(t: torch.Tensor, what: str) -> None:
    if t.device.type != "cuda":
        raise RuntimeError(
            f"{what}: expected a tensor on an AMD GPU ('cuda' device under PyTorch-ROCm), got {t.device}; "
            "flaggems_amd has no CPU implementation"
        )


def current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


# Workspace of the GEMM kernels (arrival counters, split-K partial sums, transposed scales): one zero-filled buffer
# per (device, stream), grown on demand.  Launches recorded into a HIP graph keep the raw address they were given, so
#   * a buffer that is replaced is retired, not released: a graph captured earlier may still write to it;
#   * a buffer allocated while a capture is in progress comes from that graph's private memory pool and is handed out
#     to launches of the same capture only (its zero fill is a kernel recorded in the graph; the counters are zero
#     again after every launch, so refilling them on every replay changes nothing).
# Growth at least doubles the size, so retired buffers add up to less than the live one.
_workspaces = {}   # (device index, stream handle) -> (buffer, id of the capture it was allocated in, or 0)
_retired = []


def workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    stream = torch.cuda.current_stream(device).cuda_stream
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    capture = int(load().fg_stream_capture_id(stream))
    need = max(int(nbytes), FG_WORKSPACE_COUNTER_BYTES)
    buf, made_in = _workspaces.get(key, (None, 0))
    if buf is not None and made_in not in (0, capture):
        buf = None  # belongs to another graph's pool: that graph keeps the memory, this table must not hand it out
    if buf is None or buf.numel() < need:
        if buf is not None:
            if made_in == 0:
                _retired.append(buf)
            need = max(need, 2 * buf.numel())
        buf = torch.zeros(need, dtype=torch.uint8, device=device)
        # buffers of captures that have ended stay with their graphs; this table only drops its references
        for other in [k for k, (_, cap) in _workspaces.items() if cap not in (0, capture)]:
            del _workspaces[other]
        _workspaces[key] = (buf, capture)
    return buf


def reserve_workspace(device: torch.device, nbytes: int) -> None:
    """Size the current stream's workspace ahead of time (for example before capturing a graph on this stream)."""
    workspace(torch.device(device), nbytes)
