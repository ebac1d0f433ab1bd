"""Seeded synthetic inputs for the five benchmark configurations.  Test infrastructure only.

All draws happen on a CPU generator so the CPU oracle and the GPU kernel see bit-identical inputs.
Draw order follows the reference: A then B, in their stored shapes
(iree/turbine/kernel/boo/op_exports/gemm.py:65-88); Q, K, V in argument order
(op_exports/aten.py:101-144); default seed 10 (kernel/boo/driver/driver.py:612)."""

from __future__ import annotations

import torch

DEFAULT_SEED = 10


def _gen(seed: int) -> torch.Generator:
    return torch.Generator(device="cpu").manual_seed(seed)


def gemm_inputs(M: int, N: int, K: int, seed: int = DEFAULT_SEED, std: float = 0.1, dtype: torch.dtype = torch.float16):
    """A [M, K], B [N, K] ~ N(0, 1) * std, fp16 (or `dtype`; the fp32 draws are the same either way)."""
    g = _gen(seed)
    a = (torch.randn((M, K), generator=g) * std).to(dtype)
    b = (torch.randn((N, K), generator=g) * std).to(dtype)
    return a, b


def attention_inputs(B: int, H: int, Sq: int, D: int, seed: int = DEFAULT_SEED, Sk: int | None = None):
    """Q [B, H, Sq, D]; K, V [B, H, Sk, D] ~ N(0, 1), fp16."""
    g = _gen(seed)
    Sk = Sq if Sk is None else Sk
    q = torch.randn((B, H, Sq, D), generator=g).half()
    k = torch.randn((B, H, Sk, D), generator=g).half()
    v = torch.randn((B, H, Sk, D), generator=g).half()
    return q, k, v


def paged_decode_inputs(num_seqs: int = 64, num_q_heads: int = 32, num_kv_heads: int = 8, D: int = 128, page: int = 16,
                        min_len: int = 512, max_len: int = 8192, seed: int = DEFAULT_SEED, pad_id: int = -1):
    """Context lengths uniform in [min_len, max_len]; the block table is a seeded random permutation of
    the physical pages, padded with `pad_id`; q, K cache, V cache ~ N(0, 1) fp16."""
    g = _gen(seed)
    lens = torch.randint(min_len, max_len + 1, (num_seqs,), generator=g)
    n_pg = (lens + page - 1) // page
    P = int(n_pg.sum())
    perm = torch.randperm(P, generator=g)
    max_pages = int(n_pg.max())
    bt = torch.full((num_seqs, max_pages), pad_id, dtype=torch.int32)
    off = 0
    for s in range(num_seqs):
        n = int(n_pg[s])
        bt[s, :n] = perm[off:off + n].int()
        off += n
    q = torch.randn((num_seqs, num_q_heads, D), generator=g).half()
    k_cache = torch.randn((P, page, num_kv_heads, D), generator=g).half()
    v_cache = torch.randn((P, page, num_kv_heads, D), generator=g).half()
    return q, k_cache, v_cache, bt, lens.int()


def mxfp4_inputs(M: int, N: int, K: int, seed: int = DEFAULT_SEED, exp_range: int = 8):
    """Packed E2M1 codes uniform over all 16 values, E8M0 scale bytes 127 + U[-exp_range, exp_range]."""
    g = _gen(seed)
    a = torch.randint(0, 256, (M, K // 2), generator=g).to(torch.uint8)
    a_scale = (127 + torch.randint(-exp_range, exp_range + 1, (M, K // 32), generator=g)).to(torch.uint8)
    b = torch.randint(0, 256, (N, K // 2), generator=g).to(torch.uint8)
    b_scale = (127 + torch.randint(-exp_range, exp_range + 1, (N, K // 32), generator=g)).to(torch.uint8)
    return a, a_scale, b, b_scale


def mxfp8_inputs(M: int, N: int, K: int, seed: int = DEFAULT_SEED, exp_range: int = 8):
    """E4M3 codes uniform over the 254 finite values (the two NaN patterns 0x7F / 0xFF are redrawn as their
    neighbours 0x7E / 0xFE), E8M0 scale bytes 127 + U[-exp_range, exp_range]."""
    g = _gen(seed)

    def codes(rows):
        c = torch.randint(0, 256, (rows, K), generator=g).to(torch.uint8)
        return torch.where((c & 0x7F) == 0x7F, c - 1, c)

    a = codes(M)
    a_scale = (127 + torch.randint(-exp_range, exp_range + 1, (M, K // 32), generator=g)).to(torch.uint8)
    b = codes(N)
    b_scale = (127 + torch.randint(-exp_range, exp_range + 1, (N, K // 32), generator=g)).to(torch.uint8)
    return a, a_scale, b, b_scale


def mxfp6_inputs(M: int, N: int, K: int, seed: int = DEFAULT_SEED, exp_range: int = 8):
    """6-bit codes uniform over all 64 (every code is a finite value in both formats), packed four to three
    bytes, E8M0 scale bytes 127 + U[-exp_range, exp_range].  Draw order: A codes, A scales, B codes, B scales."""
    from .mxfp6 import pack_fp6

    g = _gen(seed)
    a = torch.from_numpy(pack_fp6(torch.randint(0, 64, (M, K), generator=g)))
    a_scale = (127 + torch.randint(-exp_range, exp_range + 1, (M, K // 32), generator=g)).to(torch.uint8)
    b = torch.from_numpy(pack_fp6(torch.randint(0, 64, (N, K), generator=g)))
    b_scale = (127 + torch.randint(-exp_range, exp_range + 1, (N, K // 32), generator=g)).to(torch.uint8)
    return a, a_scale, b, b_scale
