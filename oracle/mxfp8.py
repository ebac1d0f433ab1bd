"""OCP MXFP8 (E4M3 codes + E8M0 block scales) oracle.  Test infrastructure only (see oracle/__init__.py).

The element format is the reference's `f8e4m3fn` (iree/turbine/kernel/_support/dtype.py:117-119 lists the fp8
dtypes next to the fp4 one): OCP 8-bit floating point E4M3 -- sign, 4 exponent bits (bias 7), 3 mantissa bits, no
infinities, the single NaN pattern S.1111.111, largest finite value 448.  Block scaling is the MXFP4 oracle's:
one E8M0 byte per 32 consecutive k (OCP Microscaling Formats v1.0)."""

from __future__ import annotations

import numpy as np
import torch

from .mxfp4 import BLOCK, e8m0_decode


def e4m3_closed_form(code: int) -> float:
    """Value of an 8-bit code from its bit fields."""
    s, e, m = (code >> 7) & 1, (code >> 3) & 15, code & 7
    if e == 15 and m == 7:
        return float("nan")
    mag = (m / 8.0) * 2.0 ** -6 if e == 0 else (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return -mag if s else mag


E4M3_VALUES = np.asarray([e4m3_closed_form(c) for c in range(256)], dtype=np.float32)


def mxfp8_dequant_ref(codes, scales) -> np.ndarray:
    """fp32 [rows, K]: E4M3(code) * 2^(scale - 127), scale shared by 32 consecutive k."""
    codes = codes.detach().cpu().numpy() if isinstance(codes, torch.Tensor) else np.asarray(codes)
    scales = scales.detach().cpu().numpy() if isinstance(scales, torch.Tensor) else np.asarray(scales)
    vals = E4M3_VALUES[codes.astype(np.uint8)]
    sc = np.repeat(e8m0_decode(scales), BLOCK, axis=1)
    with np.errstate(over="ignore", invalid="ignore"):
        return (vals * sc).astype(np.float32)


def mxfp8_gemm_ref(a, a_scale, b, b_scale) -> torch.Tensor:
    """fp32 matmul of the dequantised operands: C = dq(A) . dq(B)^T."""
    da = torch.from_numpy(mxfp8_dequant_ref(a, a_scale))
    db = torch.from_numpy(mxfp8_dequant_ref(b, b_scale))
    return torch.mm(da, db.t())


def mxfp8_gemm_f64(a, a_scale, b, b_scale) -> torch.Tensor:
    da = torch.from_numpy(mxfp8_dequant_ref(a, a_scale)).double()
    db = torch.from_numpy(mxfp8_dequant_ref(b, b_scale)).double()
    return torch.mm(da, db.t())


def fp8_gemm_ref(a, b, alpha: float = 1.0) -> torch.Tensor:
    """alpha . E4M3(a) . E4M3(b)^T in fp32 (no block scales).  a, b: uint8 codes or torch.float8_e4m3fn."""
    def dec(t):
        t = t.detach().cpu()
        t = t.view(torch.uint8) if t.dtype != torch.uint8 else t
        return torch.from_numpy(E4M3_VALUES[t.numpy()])
    return alpha * torch.mm(dec(a), dec(b).t())
