"""OCP MXFP6 (E2M3 or E3M2 codes + E8M0 block scales) oracle.  Test infrastructure only (see oracle/__init__.py).

The reference declares the element type `f6E2M3FN` (iree/turbine/kernel/_support/dtype.py:118) and nothing that
computes with it; the formats below are the OCP Microscaling Formats v1.0 definitions: 6 bits -- sign, then E2M3
(2 exponent bits, bias 1, 3 mantissa bits) or E3M2 (3 exponent bits, bias 3, 2 mantissa bits) -- with subnormals,
no infinities and no NaN.  Codes are packed as a little-endian bit stream per row: element k occupies bits
[6k, 6k + 6), so 4 elements take 3 bytes and a scale block of 32 takes 24."""

from __future__ import annotations

import numpy as np
import torch

from .mxfp4 import BLOCK, e8m0_decode

FORMATS = {"e2m3": (2, 3, 1), "e3m2": (3, 2, 3)}  # exponent bits, mantissa bits, bias


def fp6_closed_form(code: int, fmt: str) -> float:
    """Value of a 6-bit code from its bit fields."""
    eb, mb, bias = FORMATS[fmt]
    s, e, m = (code >> 5) & 1, (code >> mb) & ((1 << eb) - 1), code & ((1 << mb) - 1)
    mag = (m / (1 << mb)) * 2.0 ** (1 - bias) if e == 0 else (1.0 + m / (1 << mb)) * 2.0 ** (e - bias)
    return -mag if s else mag


FP6_VALUES = {f: np.asarray([fp6_closed_form(c, f) for c in range(64)], dtype=np.float32) for f in FORMATS}


def pack_fp6(codes) -> np.ndarray:
    """uint8 [rows, K*3/4] from 6-bit codes [rows, K] (K % 4 == 0): elements 4i..4i+3 -> bytes 3i..3i+2."""
    c = (codes.detach().cpu().numpy() if isinstance(codes, torch.Tensor) else np.asarray(codes)).astype(np.uint32) & 63
    rows, K = c.shape
    assert K % 4 == 0
    q = c.reshape(rows, K // 4, 4)
    word = q[:, :, 0] | (q[:, :, 1] << 6) | (q[:, :, 2] << 12) | (q[:, :, 3] << 18)  # 24 bits
    out = np.stack([word & 255, (word >> 8) & 255, (word >> 16) & 255], axis=2).astype(np.uint8)
    return out.reshape(rows, K // 4 * 3)


def unpack_fp6(packed) -> np.ndarray:
    """6-bit codes [rows, K] from the packed bytes, bit by bit (independent of pack_fp6's word arithmetic)."""
    p = packed.detach().cpu().numpy() if isinstance(packed, torch.Tensor) else np.asarray(packed)
    rows, nb = p.shape
    bits = np.unpackbits(p.astype(np.uint8), axis=1, bitorder="little")  # bit i of the row's stream
    K = nb * 8 // 6
    bits = bits[:, : K * 6].reshape(rows, K, 6).astype(np.uint8)
    return (bits << np.arange(6, dtype=np.uint8)).sum(axis=2).astype(np.uint8)


def mxfp6_dequant_ref(packed, scales, fmt: str = "e2m3") -> np.ndarray:
    """fp32 [rows, K]: FP6(code) * 2^(scale - 127), scale shared by 32 consecutive k."""
    scales = scales.detach().cpu().numpy() if isinstance(scales, torch.Tensor) else np.asarray(scales)
    vals = FP6_VALUES[fmt][unpack_fp6(packed)]
    sc = np.repeat(e8m0_decode(scales), BLOCK, axis=1)
    with np.errstate(over="ignore", invalid="ignore"):
        return (vals * sc).astype(np.float32)


def mxfp6_gemm_ref(a, a_scale, b, b_scale, fmt: str = "e2m3") -> torch.Tensor:
    """fp32 matmul of the dequantised operands: C = dq(A) . dq(B)^T."""
    da = torch.from_numpy(mxfp6_dequant_ref(a, a_scale, fmt))
    db = torch.from_numpy(mxfp6_dequant_ref(b, b_scale, fmt))
    return torch.mm(da, db.t())


def mxfp6_gemm_f64(a, a_scale, b, b_scale, fmt: str = "e2m3") -> torch.Tensor:
    da = torch.from_numpy(mxfp6_dequant_ref(a, a_scale, fmt)).double()
    db = torch.from_numpy(mxfp6_dequant_ref(b, b_scale, fmt)).double()
    return torch.mm(da, db.t())


EMAX = {"e2m3": 2, "e3m2": 4}  # exponent of the largest value: 7.5 = 1.875 * 2^2, 28 = 1.75 * 2^4


def fp6_round(y: np.ndarray, fmt: str) -> np.ndarray:
    """Magnitude code (0..31) of the value nearest to each non-negative y, by search over the value table: a tie
    goes to the even code, anything beyond the largest value to the largest value."""
    pos = FP6_VALUES[fmt][:32].astype(np.float64)
    y = np.minimum(np.asarray(y, dtype=np.float64), pos[-1])
    hi = np.clip(np.searchsorted(pos, y, side="left"), 1, 31)
    lo = hi - 1
    d_lo, d_hi = y - pos[lo], pos[hi] - y
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & (hi % 2 == 0))
    return np.where(pick_hi, hi, lo).astype(np.uint8)


def mxfp6_quantize_ref(x, fmt: str = "e2m3") -> tuple[np.ndarray, np.ndarray]:
    """(packed codes uint8 [rows, K*3/4], scales uint8 [rows, K/32]) of a [rows, K] array: OCP MX v1.0 conversion
    -- shared exponent floor(log2(max|x|)) - emax clamped to [-127, 127] (zero block: -127; NaN / infinity in the
    block: scale 0xFF, signed-zero codes); arithmetic exact in float64."""
    x = x.detach().cpu().to(torch.float64).numpy() if isinstance(x, torch.Tensor) else np.asarray(x, dtype=np.float64)
    rows, K = x.shape
    assert K % BLOCK == 0
    xb = x.reshape(rows, K // BLOCK, BLOCK)
    amax = np.abs(xb).max(axis=2)
    bad = ~np.isfinite(amax)
    with np.errstate(divide="ignore", invalid="ignore"):
        _, exp = np.frexp(np.where(bad | (amax == 0), 1.0, amax))
    shared = np.where(amax == 0, -127, np.clip(exp - 1 - EMAX[fmt], -127, 127)).astype(np.int64)
    scales = np.where(bad, 255, shared + 127).astype(np.uint8)
    y = np.abs(np.ldexp(np.where(bad[:, :, None], 0.0, xb), -shared[:, :, None]))
    code = fp6_round(y, fmt) | (np.signbit(xb).astype(np.uint8) << 5)
    return pack_fp6(code.reshape(rows, K)), scales
