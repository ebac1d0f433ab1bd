from __future__ import annotations

import torch

from .. import _lib, launch
from ..lang import sym
from ..launchable import Launchable

M, N, K = sym.M, sym.N, sym.K
BLOCK_M, BLOCK_N, BLOCK_K = sym.BLOCK_M, sym.BLOCK_N, sym.BLOCK_K

def _variant_for_tile(bm, bn) -> int:
    """First (= preferred) kernel variant of mi355_gemm_f16_nt whose tile is bm x bn; -1 (library's choice) if none."""
    if bm is None or bn is None:
        return -1
    for i, name in enumerate(_lib.variants("gemm_f16_nt")):
        if f"_{bm}x{bn}x" in name:
            return i
    return -1


def _entry(hp, a, b, c):
    variant = hp.get(sym.VARIANT)
    if variant is None:
        variant = _variant_for_tile(hp.get(BLOCK_M), hp.get(BLOCK_N))
    for s, dim, t in ((M, 0, a), (K, 1, a), (N, 0, b)):
        if s in hp and hp[s] != t.shape[dim]:
            raise ValueError(f"gemm kernel was specialised for {s}={hp[s]} but got {t.shape[dim]}")
    launch.gemm_nt_out(a, b, c, variant)


def get_gemm_kernel(shape: tuple[int, int, int], dynamic_dims: bool = False, mfma_variant=None,
                    dtype: torch.dtype = torch.float16):
    """C[M, N] = A[M, K] . B[N, K]^T with fp32 accumulation.  Call as kernel(a, b, c): a [M, K] and b [N, K] of
    `dtype` (float16 or bfloat16), c [M, N] f32 or `dtype` (written in place).

    Returns (kernel, hyperparams).  With dynamic_dims the sizes are read from the tensors at call
    time; otherwise M, N, K are bound and checked.  `mfma_variant` is accepted for call-site
    compatibility; the pre-built kernels use v_mfma_f32_32x32x16_f16 / _bf16.
    The loop nest this stands for is the TK tiled GEMM, tests/kernel/vector_codegen_test.py:71-100."""
    if dtype not in (torch.float16, torch.bfloat16):
        raise ValueError(f"get_gemm_kernel: float16 and bfloat16 operands are built, got {dtype}")
    m, n, k = shape
    if m % 256 == 0 and n % 256 == 0 and k % 64 == 0 and (m // 256) * (n // 256) >= 128:
        bm = bn = 256
    elif m % 128 == 0 and n % 128 == 0 and k % 64 == 0:
        bm = bn = 128
    else:
        bm = bn = 64
    hyperparams = {BLOCK_M: bm, BLOCK_N: bn, BLOCK_K: 64 if bm > 64 else 32}
    if not dynamic_dims:
        hyperparams.update({M: m, N: n, K: k})
    name = "gemm_bf16_nt" if dtype == torch.bfloat16 else "gemm_f16_nt"
    kernel = Launchable(name, _entry, num_outputs=1,
                        description="16-bit NT GEMM, fp32 accumulate (hand-written gfx950 MFMA kernel)")
    return kernel, hyperparams
