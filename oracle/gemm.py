"""fp16 NT GEMM oracle.  Test infrastructure only (see oracle/__init__.py)."""

from __future__ import annotations

import numpy as np
import torch


def gemm_nt_ref(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """C = A . B^T in fp32 on the CPU: `torch.mm(a, b.t())` of GEMMForward with transpose_b
    (iree/turbine/kernel/boo/op_exports/gemm.py:224-230), inputs upcast to fp32 the way the
    reference's numerics harness upcasts (kernel/boo/driver/numerics.py:94-102)."""
    return torch.mm(a.detach().cpu().float(), b.detach().cpu().float().t())


def gemm_nt_f64(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return torch.mm(a.detach().cpu().double(), b.detach().cpu().double().t())


def gemm_nt_bruteforce(a: torch.Tensor, b: torch.Tensor) -> np.ndarray:
    """Triple loop in float64 (tiny shapes only)."""
    an, bn = a.detach().cpu().double().numpy(), b.detach().cpu().double().numpy()
    M, K = an.shape
    N = bn.shape[0]
    c = np.zeros((M, N), dtype=np.float64)
    for i in range(M):
        for j in range(N):
            s = 0.0
            for k in range(K):
                s += an[i, k] * bn[j, k]
            c[i, j] = s
    return c


def gemm_nt_tiled(a: torch.Tensor, b: torch.Tensor, block_m: int = 32, block_n: int = 32, block_k: int = 32) -> torch.Tensor:
    """The loop nest of the TK tiled GEMM (tests/kernel/vector_codegen_test.py:78-100): one
    BLOCK_M x BLOCK_N accumulator per grid point, a for_loop over K tiles doing `dot`."""
    af, bf = a.detach().cpu().float(), b.detach().cpu().float()
    M, K = af.shape
    N = bf.shape[0]
    c = torch.zeros((M, N), dtype=torch.float32)
    for i in range(0, M, block_m):
        for j in range(0, N, block_n):
            acc = torch.zeros((min(block_m, M - i), min(block_n, N - j)), dtype=torch.float32)
            for k in range(0, K, block_k):
                acc = acc + af[i:i + block_m, k:k + block_k] @ bf[j:j + block_n, k:k + block_k].t()
            c[i:i + block_m, j:j + block_n] = acc
    return c
