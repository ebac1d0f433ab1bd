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
