"""FP8 (OCP e4m3fn) row-wise quantisation oracle (numpy, bit level).

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

Restates /root/reference/kernels/pytorch/quant_fp8.py:13-40 and the quantisers
of /root/reference/kernels/pytorch/moe_fp8.py:17-43.  The e4m3fn cast, which the
reference delegates to ``Tensor.to(torch.float8_e4m3fn)``, is restated on the
bit pattern so that it can be checked against that library routine instead of
being it.
"""
from __future__ import annotations

import numpy as np

FP8_MAX = 448.0           # quant_fp8.py:16
SCALE_CLAMP = 2.0 ** 127  # quant_fp8.py:23


def e4m3fn_decode_table() -> np.ndarray:
    """float32 value of each of the 256 e4m3fn codes (1-4-3, bias 7, no inf,
    S.1111.111 = NaN)."""
    out = np.zeros(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp = (code >> 3) & 0xF
        man = code & 0x7
        if exp == 0xF and man == 0x7:
            val = float("nan")
        elif exp == 0:
            val = sign * man * 2.0 ** -9
        else:
            val = sign * (1.0 + man / 8.0) * 2.0 ** (exp - 7)
        out[code] = val
    return out


_DECODE = e4m3fn_decode_table()


def e4m3fn_decode(codes: np.ndarray) -> np.ndarray:
    return _DECODE[np.asarray(codes, dtype=np.uint8)]


def e4m3fn_encode(x: np.ndarray) -> np.ndarray:
    """float32 -> e4m3fn code, round-to-nearest-even, NON-saturating: any value
    whose rounded magnitude exceeds 448 (and inf, NaN) becomes the NaN code
    ``sign|0x7F`` -- the behaviour of ``Tensor.to(torch.float8_e4m3fn)`` that
    quant_fp8.py:33 relies on."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    mag = np.abs(x).astype(np.float64)
    out = np.zeros(x.shape, dtype=np.uint8)

    finite = np.isfinite(x)
    # quantum of the target grid: 2^-9 below 2^-6 (subnormals), else 2^(e-3)
    with np.errstate(divide="ignore", invalid="ignore"):
        e = np.floor(np.log2(np.where(mag > 0, mag, 1.0)))
    e = np.maximum(e, -6.0)
    quantum = np.exp2(e - 3.0)
    with np.errstate(invalid="ignore"):
        steps = mag / quantum                   # exact: power-of-two divisor
        r = np.rint(steps)                      # numpy rint = ties to even
        val = r * quantum                       # rounded magnitude (may carry into next binade)
    # re-derive exponent/mantissa of the rounded magnitude
    with np.errstate(divide="ignore", invalid="ignore"):
        e2 = np.floor(np.log2(np.where(val > 0, val, 1.0)))
    with np.errstate(invalid="ignore"):
        sub = val < 2.0 ** -6
        man_sub = np.rint(val / 2.0 ** -9)
        exp_n = e2 + 7.0
        man_n = np.rint((val / np.exp2(e2) - 1.0) * 8.0)
        code = np.where(sub, man_sub, exp_n * 8.0 + man_n)
        overflow = (val > FP8_MAX) | ~finite
        code = np.where(overflow, 0x7F, code)
    out = code.astype(np.uint8) | sign
    return out


def calculate_scale(a_max: np.ndarray, dtype: str = "fp32") -> np.ndarray:
    """Power-of-two multiplier ``exp2(floor(log2(448 / amax)))`` (quant_fp8.py:13-24).

    ``448 / amax`` is evaluated in the input's dtype before the cast to fp32
    (quant_fp8.py:17): for bf16 inputs the quotient is rounded to bf16.  ``log2``
    is the fp32 one of the reference formula, taken here as the correctly rounded
    value (float64 log2 rounded to float32).  That matters for fp32 inputs only:
    a quotient within ~1e-6 below a power of two has an fp32 log2 that rounds UP
    to the integer, so the formula returns the larger power of two; a quotient of
    a bf16 amax never comes that close.  NaN or +-inf results are replaced by
    2^127 (:19-23); amax = inf gives quotient 0 and scale 0 (finite, so kept)."""
    from .routing import round_to_bf16

    a_max = np.asarray(a_max, dtype=np.float32)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        q = (np.float32(FP8_MAX) / a_max).astype(np.float32)
        if dtype == "bf16":
            q = round_to_bf16(q)
        elif dtype != "fp32":
            raise ValueError(dtype)
        lg = np.log2(q.astype(np.float64)).astype(np.float32)
        scale = np.exp2(np.floor(lg).astype(np.float64)).astype(np.float32)
    bad = ~np.isfinite(scale)
    scale[bad] = np.float32(SCALE_CLAMP)
    return scale


def rowwise_quant_fp8(a: np.ndarray, dtype: str = "fp32"):
    """Row-wise (last dim) quantisation (quant_fp8.py:27-34).

    a : [..., n] float32 holding values representable in ``dtype``.
    Returns ``(codes uint8 [..., n], scale float32 [...])`` with
    ``codes = e4m3fn(a * scale)`` and ``scale`` the MULTIPLIER."""
    a = np.asarray(a, dtype=np.float32)
    if a.shape[-1] == 0:
        raise ValueError("rowwise quant needs at least one column")
    a_max = np.max(np.abs(a), axis=-1)
    # torch.max propagates NaN; numpy max does too
    scale = calculate_scale(a_max, dtype)
    with np.errstate(over="ignore", invalid="ignore"):
        scaled = (a * scale[..., None]).astype(np.float32)
    return e4m3fn_encode(scaled), scale


def transpose_rowwise_quant_fp8(a: np.ndarray, dtype: str = "fp32"):
    """quant_fp8.py:37-40: quantise ``a.transpose(-2, -1)`` row-wise."""
    return rowwise_quant_fp8(np.swapaxes(np.asarray(a), -2, -1), dtype)


def silu_f32(x: np.ndarray) -> np.ndarray:
    x = np.asarray(x, dtype=np.float32)
    with np.errstate(over="ignore"):
        return (x / (np.float32(1.0) + np.exp(-x).astype(np.float32))).astype(np.float32)


def silu_bf16(x: np.ndarray) -> np.ndarray:
    """F.silu on a bf16 tensor: x / (1 + exp(-x)) evaluated in fp32 and rounded to bf16.  A function
    of 65536 inputs, fixed here independently of any library's last-place error in exp: the
    quotient in float64, rounded to fp32 and then to bf16; where exp(-x) overflows fp32 (x below
    -log(FLT_MAX) = -88.72) the fp32 formula divides by infinity: -0, and NaN for x = -inf.
    Pinned on all 65536 inputs against torch's CPU kernel and against silu_f32 + rounding."""
    from .routing import round_to_bf16

    x = np.asarray(x, dtype=np.float32)
    x64 = x.astype(np.float64)
    with np.errstate(over="ignore", invalid="ignore"):
        y = (x64 / (1.0 + np.exp(-x64))).astype(np.float32)
        over = -x64 > np.log(np.float64(np.finfo(np.float32).max))
        y = np.where(over, (x64 / np.inf).astype(np.float32), y)      # -0, and NaN for x = -inf
    return round_to_bf16(y)


def silu_rowwise_quant_fp8(a: np.ndarray, dtype: str = "fp32"):
    """moe_fp8.py:17-33: SiLU in the input dtype, upcast, row-wise scale from the
    fp32 amax (``calculate_scale`` then sees an fp32 tensor), e4m3fn cast."""
    s = silu_bf16(a) if dtype == "bf16" else silu_f32(a)
    return rowwise_quant_fp8(s, "fp32")


def bmm_weight_rowwise_quant_fp8(weight: np.ndarray, dtype: str = "fp32"):
    """moe_fp8.py:36-43: weight [E, D_in, D_out], amax over D_in (dim 1) per
    (expert, output column); returns codes [E, D_in, D_out] and scale [E, D_out]."""
    w = np.asarray(weight, dtype=np.float32)
    a_max = np.max(np.abs(w), axis=1)
    scale = calculate_scale(a_max, dtype)
    with np.errstate(over="ignore", invalid="ignore"):
        scaled = (w * scale[:, None, :]).astype(np.float32)
    return e4m3fn_encode(scaled), scale
