"""OCP FP8 E4M3FN codec written from the format definition (numpy, CPU only).

TEST INFRASTRUCTURE. Only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this module; the product path never does.

Format (OCP 8-bit Floating Point Specification, "E4M3"): 1 sign bit, 4 exponent
bits with bias 7, 3 mantissa bits, no infinities, a single NaN mantissa pattern
(S.1111.111), largest finite value S.1111.110 = 448, smallest subnormal
2**-9.  Conversion from wider types is round-to-nearest-even; values whose
rounded magnitude exceeds 448 become NaN (this is what
``tensor.to(torch.float8_e4m3fn)`` does: it does not saturate), NaN keeps its
sign bit, +-Inf become NaN.

The encoder below is used to pin the torch-based oracle
(``oracle/fp8_linear_oracle.py``): tests compare it with
``tensor.to(torch.float8_e4m3fn)`` over every bf16 bit pattern, and the
brute-force quantizer in the tests is built on it.
"""
from __future__ import annotations

import numpy as np

E4M3_MAX = 448.0
E4M3_MIN_SUBNORMAL = 2.0 ** -9
E4M3_MIN_NORMAL = 2.0 ** -6


def decode_table() -> np.ndarray:
    """float32 value of each of the 256 codes (NaN for 0x7F and 0xFF)."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp = (code >> 3) & 0xF
        man = code & 0x7
        if exp == 0xF and man == 0x7:
            val = float("nan")
        elif exp == 0:
            val = sign * man * 2.0 ** -9  # subnormal: 0.mmm * 2**-6
        else:
            val = sign * (1.0 + man / 8.0) * 2.0 ** (exp - 7)
        out[code] = val
    return out


_DECODE = decode_table()


def decode(codes: np.ndarray) -> np.ndarray:
    return _DECODE[np.asarray(codes, dtype=np.uint8)]


def encode(values: np.ndarray) -> np.ndarray:
    """float32 -> E4M3FN code, round-to-nearest-even, overflow -> NaN.

    Works in float64 so every intermediate is exact: a float32 scaled by a power
    of two and rounded to an integer with ``np.rint`` (ties-to-even).
    """
    v = np.asarray(values, dtype=np.float32)
    bits = v.view(np.uint32)
    sign = ((bits >> 31) & 1).astype(np.uint8) << 7
    a = np.abs(v.astype(np.float64))
    out = np.zeros(v.shape, dtype=np.uint8)

    nan_like = ~np.isfinite(a)
    finite = ~nan_like

    # Exponent of the target binade, clamped below at the subnormal binade (-6).
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where((a > 0) & finite, a, 1.0)))
    e = np.maximum(e, -6.0)
    # Quantum in that binade is 2**(e-3); round to an integer number of quanta.
    q = np.rint(np.where(finite, a, 0.0) / np.exp2(e - 3.0))
    # Rounding may carry into the next binade (q == 16).
    carry = q >= 16
    e = np.where(carry, e + 1.0, e)
    q = np.where(carry, 8.0, q)

    normal = q >= 8
    exp_field = np.where(normal, e + 7.0, 0.0)
    man_field = np.where(normal, q - 8.0, q)
    mag = (exp_field.astype(np.int64) << 3) | man_field.astype(np.int64)
    overflow = (exp_field > 15) | (mag > 0x7E)
    mag = np.where(overflow | nan_like, 0x7F, mag)
    out = sign | mag.astype(np.uint8)
    return out


def encode_scalar_reference(x: float) -> int:
    """Slow, independent encoder: pick the nearest representable value by search.

    Used only to cross-check ``encode`` on small inputs.  Ties go to the code with
    an even mantissa field; magnitudes that would round above 448 (>= 464, the
    midpoint to the next would-be value 480) give NaN.
    """
    import math

    if math.isnan(x):
        return 0xFF if math.copysign(1.0, x) < 0 else 0x7F
    s = 0x80 if math.copysign(1.0, x) < 0 else 0
    a = abs(x)
    if math.isinf(a) or a > 464.0:
        return s | 0x7F
    best, best_err = 0, None
    for code in range(0x7F):  # positive finite codes 0x00..0x7E
        err = abs(float(_DECODE[code]) - a)
        if best_err is None or err < best_err or (err == best_err and code % 2 == 0):
            best, best_err = code, err
    if a == 464.0:
        # Tie between 448 (mantissa 110, even) and the absent 480 (would be 111).
        return s | 0x7E
    return s | best
