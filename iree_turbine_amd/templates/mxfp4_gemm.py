from __future__ import annotations

from .. import launch
from ..lang import sym
from ..launchable import Launchable

M, N, K = sym.M, sym.N, sym.K
BLOCK_M, BLOCK_N, BLOCK_K = sym.BLOCK_M, sym.BLOCK_N, sym.BLOCK_K


def _entry(hp, a, a_scale, b, b_scale, c):
    for s, got in ((M, a.shape[0]), (N, b.shape[0]), (K, a.shape[1] * 2)):
        if s in hp and hp[s] != got:
            raise ValueError(f"mxfp4 gemm kernel was specialised for {s}={hp[s]} but got {got}")
    launch.mxfp4_gemm_out(a, a_scale, b, b_scale, c, hp.get(sym.VARIANT, -1))


def get_mxfp4_gemm_kernel(shape: tuple[int, int, int], dynamic_dims: bool = False, mfma_variant=None):
    """C[M, N] = dq(A) . dq(B)^T for MXFP4 operands (scaled MFMA, F32_32x32x64_F8F6F4 with fp4 inputs).
    Call as kernel(a, a_scale, b, b_scale, c): a u8 [M, K/2], a_scale u8 [M, K/32], b u8 [N, K/2],
    b_scale u8 [N, K/32], c bf16 or f32 [M, N] (written in place).  Two E2M1 codes per byte, even k
    in the low nibble; one E8M0 scale per 32 k.  Element types: f4e2m1fn / f8e8m0fnu,
    iree/turbine/kernel/_support/dtype.py:117,119.  Returns (kernel, hyperparams)."""
    m, n, k = shape
    if k % 32:
        raise ValueError(f"get_mxfp4_gemm_kernel: K={k} must be a multiple of 32")
    big = m % 256 == 0 and n % 256 == 0 and k % 256 == 0 and (m // 256) * (n // 256) >= 128
    mid = m % 128 == 0 and n % 128 == 0 and k % 256 == 0
    hyperparams = {BLOCK_M: 256 if big else 128 if mid else 32, BLOCK_N: 256 if big else 128, BLOCK_K: 256 if (big or mid) else 64}
    if not dynamic_dims:
        hyperparams.update({M: m, N: n, K: k})
    return Launchable("mxfp4_gemm", _entry, num_outputs=1, description="block-scaled MXFP4 GEMM (gfx950 scaled MFMA)"), hyperparams
