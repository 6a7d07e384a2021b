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
    "fg_inv_rope_group_quant_fp8": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p, c_int64, c_int64,
         c_int64, c_int64, c_int64, c_float, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p],
    ),
    "fg_silu_mul": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p]),
    "fg_moe_sum": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p]),
    "fg_topk_softmax": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p]),
    "fg_grouped_topk": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int, c_float, c_int,
                                c_void_p, c_void_p, c_int64, c_void_p]),
    "fg_moe_sort_slots": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p, c_void_p, c_void_p]),
    "fg_moe_align_block_size": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p]),
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


_fast = None
_addresses = {}


def fast():
    """The CPython marshalling module for the decode-critical calls (csrc/fastcall.c, built next to the library by
    flaggems_amd/build.py).  A ctypes call converts its 20-odd arguments in 2-3 us, as long as a decode kernel runs;
    this module takes the function's address and the arguments as plain Python ints and floats."""
    global _fast
    if _fast is None:
        import importlib.util

        from .build import fastcall_path

        path = fastcall_path()
        if not os.path.exists(path):
            raise ImportError(f"{path} is missing: build it with `python -m flaggems_amd.build`")
        spec = importlib.util.spec_from_file_location("_fg_fastcall", path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _fast = mod
    return _fast


def address(name: str) -> int:
    """Address of an exported C function, for the calls that go through `fast()`."""
    a = _addresses.get(name)
    if a is None:
        a = ctypes.cast(getattr(load(), name), c_void_p).value
        _addresses[name] = a
    return a


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


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream_ptr(device: torch.device) -> int:
    """The hipStream_t of torch's current stream on ``device`` (the raw getter skips building a Stream object, which
    costs more host time than everything else the wrappers do around a launch)."""
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()
_single_gpu = None  # this process sees exactly one GPU (asked once): there is no other device to guard against


def device_guard(device: torch.device):
    """``torch.cuda.device(device)``, or nothing at all when that device is already the current one (the usual case:
    entering and leaving the context manager costs more host time than a decode-sized launch)."""
    global _single_gpu
    if _single_gpu is None:
        _single_gpu = torch.cuda.device_count() == 1
    if _single_gpu or device.index is None or device.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)


_ws_bytes_cache = {}


def cached_workspace_bytes(fn_name: str, *shape) -> int:
    """``lib.<fn_name>(*shape)``, remembered per shape (the answer depends on the shape and the device's compute unit
    count only; processes that mix GPU models would have to clear the table)."""
    key = (fn_name, shape)
    n = _ws_bytes_cache.get(key)
    if n is None:
        n = int(getattr(load(), fn_name)(*shape))
        if len(_ws_bytes_cache) > 4096:
            _ws_bytes_cache.clear()
        _ws_bytes_cache[key] = n
    return n


# Workspace of the GEMM kernels (arrival counters, split-K partial sums, transposed scales): one buffer per
# (device, stream) whose first FG_WORKSPACE_COUNTER_BYTES are zero, grown on demand.  Only the counter area needs the
# zeros (every launch leaves it zero again); partial sums and transposed scales are written before they are read.
# Launches recorded into a HIP graph keep the raw address they were given, so
#   * a buffer that is replaced is retired, not released: a graph captured earlier may still write to it;
#   * a buffer allocated while a capture is in progress comes from that graph's private memory pool and is handed out
#     to launches of the same capture only.  The fill of its counter area is a 16 KB kernel recorded in the graph,
#     which every replay repeats; `reserve_workspace()` on the capture stream before the capture avoids even that.
# Growth at least doubles the size, so retired buffers add up to less than the live one; the list keeps the most
# recent kMaxRetired of them (a graph that still uses an older one than that would have to be older than that many
# growth steps of one stream).
_workspaces = {}   # (device index, stream handle) -> (buffer, id of the capture it was allocated in, or 0)
_retired = []
kMaxRetired = 64


def _capture_id(stream: int) -> int:
    """0 unless the current stream is being captured into a graph (then the capture's id)."""
    if not torch.cuda.is_current_stream_capturing():
        return 0
    return int(load().fg_stream_capture_id(stream))


def workspace(device: torch.device, nbytes: int, stream: int = None) -> torch.Tensor:
    if stream is None:
        stream = current_stream_ptr(device)
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    capture = _capture_id(stream)
    need = max(int(nbytes), FG_WORKSPACE_COUNTER_BYTES)
    buf, made_in = _workspaces.get(key, (None, 0))
    if buf is not None and made_in == capture and buf.numel() >= need:
        return buf
    if buf is not None and made_in not in (0, capture):
        buf = None  # belongs to another graph's pool: that graph keeps the memory, this table must not hand it out
    if buf is None or buf.numel() < need:
        if buf is not None:
            if made_in == 0:
                _retired.append(buf)
                del _retired[:-kMaxRetired]
            need = max(need, 2 * buf.numel())
        buf = torch.empty(need, dtype=torch.uint8, device=device)
        buf[:FG_WORKSPACE_COUNTER_BYTES].zero_()
        # buffers of captures that have ended stay with their graphs; this table only drops its references
        for other in [k for k, (_, cap) in _workspaces.items() if cap not in (0, capture)]:
            del _workspaces[other]
        _workspaces[key] = (buf, capture)
    return buf


def reserve_workspace(device: torch.device, nbytes: int) -> None:
    """Size the current stream's workspace ahead of time (for example before capturing a graph on this stream)."""
    workspace(torch.device(device), nbytes)
