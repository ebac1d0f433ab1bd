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
