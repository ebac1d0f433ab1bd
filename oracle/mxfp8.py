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


E4M3_EMAX = 8  # exponent of the largest finite E4M3 value, 448 = 1.75 * 2^8
_POS = E4M3_VALUES[:127].astype(np.float64)  # codes 0x00..0x7E ascend in value; 0x7F is NaN


def e4m3_round(y: np.ndarray) -> np.ndarray:
    """Code (0..0x7E) of the E4M3 value nearest to each non-negative y, by search over the value table: a tie
    goes to the even code, anything beyond 448 to 448."""
    y = np.minimum(np.asarray(y, dtype=np.float64), _POS[-1])
    hi = np.clip(np.searchsorted(_POS, y, side="left"), 1, len(_POS) - 1)
    lo = hi - 1
    d_lo, d_hi = y - _POS[lo], _POS[hi] - y
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & (hi % 2 == 0))
    return np.where(pick_hi, hi, lo).astype(np.uint8)


def mxfp8_quantize_ref(x) -> tuple[np.ndarray, np.ndarray]:
    """(codes uint8 [rows, K], scales uint8 [rows, K/32]) of a [rows, K] array: OCP MX v1.0 conversion with E4M3
    elements -- shared exponent floor(log2(max|x|)) - 8 clamped to [-127, 127] (zero block: -127; NaN / infinity
    in the block: scale 0xFF, signed-zero codes); arithmetic exact in float64."""
    x = x.detach().cpu().to(torch.float64).numpy() if isinstance(x, torch.Tensor) else np.asarray(x, dtype=np.float64)
    rows, K = x.shape
    assert K % BLOCK == 0
    xb = x.reshape(rows, K // BLOCK, BLOCK)
    amax = np.abs(xb).max(axis=2)
    bad = ~np.isfinite(amax)
    with np.errstate(divide="ignore", invalid="ignore"):
        _, exp = np.frexp(np.where(bad | (amax == 0), 1.0, amax))
    shared = np.where(amax == 0, -127, np.clip(exp - 1 - E4M3_EMAX, -127, 127)).astype(np.int64)
    scales = np.where(bad, 255, shared + 127).astype(np.uint8)
    y = np.abs(np.ldexp(np.where(bad[:, :, None], 0.0, xb), -shared[:, :, None]))
    code = e4m3_round(y) | (np.signbit(xb).astype(np.uint8) << 7)
    return code.reshape(rows, K), scales
