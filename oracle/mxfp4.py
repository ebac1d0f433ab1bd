"""OCP MXFP4 (E2M1 codes + E8M0 block scales) oracle.  Test infrastructure only (see oracle/__init__.py)."""

from __future__ import annotations

import numpy as np
import torch

# OCP Microscaling Formats v1.0, FP4 E2M1: sign bit 3, exponent bits 2:1 (bias 1), mantissa bit 0.
E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0)
BLOCK = 32  # elements sharing one E8M0 scale


def e2m1_closed_form(code: int) -> float:
    """Value of a 4-bit code from the bit fields (independent of the table above)."""
    s, e, m = (code >> 3) & 1, (code >> 1) & 3, code & 1
    mag = (m * 0.5) if e == 0 else (1.0 + 0.5 * m) * 2.0 ** (e - 1)
    return -mag if s else mag


def e8m0_decode(b: np.ndarray) -> np.ndarray:
    """2^(b - 127) as fp32; 0xFF is NaN."""
    b = np.asarray(b, dtype=np.uint8)
    out = np.ldexp(np.float32(1.0), np.minimum(b, 254).astype(np.int32) - 127).astype(np.float32)
    out[b == 255] = np.nan
    return out


def unpack_codes(packed: np.ndarray) -> np.ndarray:
    """uint8 [rows, K/2] -> uint8 [rows, K]; element 2i is the low nibble of byte i."""
    packed = np.asarray(packed, dtype=np.uint8)
    out = np.empty((packed.shape[0], packed.shape[1] * 2), dtype=np.uint8)
    out[:, 0::2] = packed & 0xF
    out[:, 1::2] = packed >> 4
    return out


def pack_codes(codes: np.ndarray) -> np.ndarray:
    codes = np.asarray(codes, dtype=np.uint8)
    return (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)


def mxfp4_dequant_ref(packed, scales) -> np.ndarray:
    """fp32 [rows, K]: E2M1(code) * 2^(scale - 127), scale shared by 32 consecutive k."""
    packed = packed.detach().cpu().numpy() if isinstance(packed, torch.Tensor) else np.asarray(packed)
    scales = scales.detach().cpu().numpy() if isinstance(scales, torch.Tensor) else np.asarray(scales)
    vals = np.asarray(E2M1_VALUES, dtype=np.float32)[unpack_codes(packed)]
    sc = np.repeat(e8m0_decode(scales), BLOCK, axis=1)
    with np.errstate(over="ignore", invalid="ignore"):
        return (vals * sc).astype(np.float32)


def mxfp4_gemm_ref(a, a_scale, b, b_scale) -> torch.Tensor:
    """fp32 matmul of the dequantised operands: C = dq(A) . dq(B)^T."""
    da = torch.from_numpy(mxfp4_dequant_ref(a, a_scale))
    db = torch.from_numpy(mxfp4_dequant_ref(b, b_scale))
    return torch.mm(da, db.t())


def mxfp4_gemm_f64(a, a_scale, b, b_scale) -> torch.Tensor:
    da = torch.from_numpy(mxfp4_dequant_ref(a, a_scale)).double()
    db = torch.from_numpy(mxfp4_dequant_ref(b, b_scale)).double()
    return torch.mm(da, db.t())


# ---- quantisation (OCP Microscaling Formats v1.0, section 6.3: conversion to an MX block) -----------------
# For every block of 32 consecutive k:  shared exponent = floor(log2(max |x|)) - emax(E2M1 = 2), clamped
# to the E8M0 range [-127, 127]; every element is divided by 2^shared (exact) and rounded to the nearest
# E2M1 value, ties to the even code, magnitudes beyond 6 saturate to 6.  A block holding a NaN or an
# infinity gets the NaN scale 0xFF and zero magnitudes (signs kept).  An all-zero block gets the smallest
# scale (byte 0).

E2M1_EMAX = 2
_E2M1_MAGS = np.asarray(E2M1_VALUES[:8], dtype=np.float64)


def e2m1_round_brute_force(y: float) -> int:
    """Magnitude code (0..7) of the E2M1 value nearest to y >= 0; of two equally near values the one with
    the even code; beyond 6 -> 7.  Exhaustive search, independent of any threshold table."""
    best, best_d = 0, abs(y - _E2M1_MAGS[0])
    for c in range(1, 8):
        d = abs(y - _E2M1_MAGS[c])
        if d < best_d or (d == best_d and c % 2 == 0 and best % 2 == 1):
            best, best_d = c, d
    return best


def mxfp4_quantize_ref(x) -> tuple[np.ndarray, np.ndarray]:
    """(codes uint8 [rows, K/2], scales uint8 [rows, K/32]) of a [rows, K] array (any float dtype; the
    arithmetic is exact in float64)."""
    x = x.detach().cpu().to(torch.float64).numpy() if isinstance(x, torch.Tensor) else np.asarray(x, dtype=np.float64)
    rows, K = x.shape
    assert K % BLOCK == 0
    xb = x.reshape(rows, K // BLOCK, BLOCK)
    amax = np.abs(xb).max(axis=2)
    bad = ~np.isfinite(amax)
    with np.errstate(divide="ignore", invalid="ignore"):
        mant, exp = np.frexp(np.where(bad | (amax == 0), 1.0, amax))   # amax = mant * 2^exp, mant in [0.5, 1)
    shared = np.where(amax == 0, -127, np.clip(exp - 1 - E2M1_EMAX, -127, 127)).astype(np.int64)
    scales = np.where(bad, 255, shared + 127).astype(np.uint8)
    y = np.abs(np.ldexp(np.where(bad[:, :, None], 0.0, xb), -shared[:, :, None]))
    # thresholds halfway between neighbours; a tie goes to the even code
    code = ((y > 0.25).astype(np.uint8) + (y >= 0.75) + (y > 1.25) + (y >= 1.75) + (y > 2.5) + (y >= 3.5) + (y > 5.0)).astype(np.uint8)
    code |= (np.signbit(xb).astype(np.uint8) << 3)
    return pack_codes(code.reshape(rows, K)), scales
