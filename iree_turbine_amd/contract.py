"""The shape / dtype contract of the kernels, as host-side checks on tensors (real or meta).

Both routes to the C ABI run them: the custom ops in their `select` (which is also their Meta kernel) and
the out-variant launchers that the template kernels call directly.  A violation raises ValueError before
anything is launched; what the checks let through is what the kernels' address arithmetic assumes, so a
short operand can never become an out-of-bounds device access.
"""

from __future__ import annotations

import torch
from torch import Tensor

HALF_DTYPES = (torch.float16, torch.bfloat16)  # the attention and GEMM kernels are built for both 16-bit formats
PAGE_SIZES = (16, 32, 64, 128, 256)  # tokens per KV-cache page


def require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def same_half_dtype(tensors) -> bool:
    return tensors[0].dtype in HALF_DTYPES and all(t.dtype == tensors[0].dtype for t in tensors)


def check_gemm_operands(op: str, a: Tensor, b: Tensor, dtypes=HALF_DTYPES, what: str = "float16 or both bfloat16") -> None:
    require(a.dim() == 2 and b.dim() == 2, f"{op}: a and b must be rank 2")
    require(a.dtype in dtypes and b.dtype in dtypes and (a.dtype == b.dtype or dtypes is not HALF_DTYPES),
            f"{op}: a and b must both be {what}, got {a.dtype} and {b.dtype}")
    require(a.size(1) == b.size(1), f"{op}: K mismatch, a is {tuple(a.shape)}, b is {tuple(b.shape)} (b is [N, K])")
    require(a.size(0) > 0 and b.size(0) > 0 and a.size(1) > 0, f"{op}: empty operand")


def check_attention_operands(op: str, q: Tensor, k: Tensor, v: Tensor) -> None:
    for name, t in (("q", q), ("k", k), ("v", v)):
        require(t.dim() == 4, f"{op}: {name} must be [B, H, S, D]")
    require(same_half_dtype((q, k, v)), f"{op}: q, k, v must all be float16 or all bfloat16")
    require(q.size(3) == 128, f"{op}: head dim {q.size(3)} not supported (only 128)")
    require(k.shape == v.shape, f"{op}: k and v shapes differ")
    require(q.size(0) == k.size(0) and q.size(3) == k.size(3), f"{op}: q and k disagree on B or D")
    require(k.size(1) > 0 and q.size(1) % k.size(1) == 0, f"{op}: {q.size(1)} query heads over {k.size(1)} key/value heads")
    require(q.size(2) > 0 and k.size(2) > 0, f"{op}: empty sequence")


def check_block_table(op: str, block_table: Tensor, per_seq: Tensor, num_seqs: int, per_seq_name: str = "seq_lens") -> None:
    """block_table int32 [num_seqs, max_pages] and a per-sequence int32 vector (an int64 tensor, torch's default
    for integer data, would be read as twice as many half-sized values)."""
    require(block_table.dim() == 2 and block_table.dtype == torch.int32, f"{op}: block_table must be int32 [num_seqs, max_pages_per_seq], got {block_table.dtype} {tuple(block_table.shape)}")
    require(per_seq.dim() == 1 and per_seq.dtype == torch.int32, f"{op}: {per_seq_name} must be int32 [num_seqs], got {per_seq.dtype} {tuple(per_seq.shape)}")
    require(block_table.size(0) == num_seqs and per_seq.size(0) == num_seqs, f"{op}: block_table / {per_seq_name} rows must equal num_seqs = {num_seqs}")
    require(num_seqs > 0 and block_table.size(1) > 0, f"{op}: empty batch")


def check_paged_args(op: str, q: Tensor, k_cache: Tensor, v_cache: Tensor, block_table: Tensor, seq_lens: Tensor,
                     bf16_ok: bool = False) -> None:
    require(q.dim() == 3, f"{op}: q must be [num_seqs, num_q_heads, D]")
    require(k_cache.dim() == 4 and v_cache.shape == k_cache.shape, f"{op}: k_cache / v_cache must both be [num_pages, page_size, num_kv_heads, D]")
    if bf16_ok:
        require(same_half_dtype((q, k_cache, v_cache)), f"{op}: q, k_cache, v_cache must all be float16 or all bfloat16")
    else:
        require(q.dtype == torch.float16 and k_cache.dtype == torch.float16 and v_cache.dtype == torch.float16, f"{op}: q, k_cache, v_cache must be float16")
    check_block_table(op, block_table, seq_lens, q.size(0))
    require(q.size(2) == 128 and k_cache.size(3) == 128, f"{op}: head dim must be 128")
    require(k_cache.size(1) in PAGE_SIZES, f"{op}: page size {k_cache.size(1)} not supported {PAGE_SIZES}")
    hq, hkv = q.size(1), k_cache.size(2)
    require(hkv > 0 and hq % hkv == 0 and hq // hkv in (1, 2, 4, 8, 16), f"{op}: {hq} q heads over {hkv} kv heads is not supported (ratio 1, 2, 4, 8 or 16)")
    require(k_cache.size(0) > 0, f"{op}: empty cache")


def check_decode_partials(op: str, part_acc: Tensor, part_ml: Tensor, num_seqs: int, num_q_heads: int, splits: int | None = None) -> int:
    """part_acc fp32 [S, Hq, splits, 128] and part_ml fp32 [S, Hq, splits, 2]; returns the split count."""
    require(part_acc.dim() == 4 and part_acc.dtype == torch.float32 and part_ml.dtype == torch.float32,
            f"{op}: part_acc must be fp32 [S, Hq, splits, 128], part_ml fp32 [S, Hq, splits, 2]")
    ns = part_acc.size(2) if splits is None else splits
    require(tuple(part_acc.shape) == (num_seqs, num_q_heads, ns, 128) and tuple(part_ml.shape) == (num_seqs, num_q_heads, ns, 2),
            f"{op}: part_acc must be fp32 {(num_seqs, num_q_heads, ns, 128)} and part_ml fp32 {(num_seqs, num_q_heads, ns, 2)}, got "
            f"{tuple(part_acc.shape)} and {tuple(part_ml.shape)}")
    require(1 <= ns <= 1024, f"{op}: the number of kv splits must be in [1, 1024], got {ns}")
    return ns


def check_kv_append(op: str, k_new: Tensor, v_new: Tensor, k_cache: Tensor, v_cache: Tensor, block_table: Tensor, start_pos: Tensor) -> None:
    require(k_new.dim() == 4 and k_new.shape == v_new.shape, f"{op}: k_new and v_new must both be [S, n_new, Hkv, D]")
    require(k_cache.dim() == 4 and k_cache.shape == v_cache.shape, f"{op}: k_cache and v_cache must both be [P, page, Hkv, D]")
    require(same_half_dtype((k_new, v_new, k_cache, v_cache)), f"{op}: tensors must all be float16 or all bfloat16")
    require(k_new.size(3) == 128 and k_cache.size(3) == 128, f"{op}: head dim must be 128")
    require(k_cache.size(1) in PAGE_SIZES, f"{op}: page size {k_cache.size(1)} not supported {PAGE_SIZES}")
    require(k_new.size(2) == k_cache.size(2), f"{op}: k_new and k_cache disagree on the number of kv heads")
    require(k_new.size(0) > 0 and k_new.size(1) > 0 and k_cache.size(0) > 0, f"{op}: empty k_new or cache")
    check_block_table(op, block_table, start_pos, k_new.size(0), "start_pos")


def check_paged_prefill(op: str, q: Tensor, k_cache: Tensor, v_cache: Tensor, block_table: Tensor, seq_lens: Tensor) -> None:
    require(q.dim() == 4, f"{op}: q must be [num_seqs, n_new, num_q_heads, D]")
    require(k_cache.dim() == 4 and k_cache.shape == v_cache.shape, f"{op}: k_cache / v_cache must both be [num_pages, page_size, num_kv_heads, D]")
    require(same_half_dtype((q, k_cache, v_cache)), f"{op}: q, k_cache, v_cache must all be float16 or all bfloat16")
    require(q.size(3) == 128 and k_cache.size(3) == 128, f"{op}: head dim must be 128")
    require(k_cache.size(1) in PAGE_SIZES, f"{op}: page size {k_cache.size(1)} not supported {PAGE_SIZES}")
    require(k_cache.size(2) > 0 and q.size(2) % k_cache.size(2) == 0, f"{op}: {q.size(2)} q heads over {k_cache.size(2)} kv heads")
    check_block_table(op, block_table, seq_lens, q.size(0))
    require(q.size(1) > 0 and k_cache.size(0) > 0, f"{op}: empty batch")


def check_mx_operand(op: str, name: str, codes: Tensor, scales: Tensor, per_byte: int = 2) -> int:
    """codes uint8 [rows, K / per_byte] with scales uint8 [rows, K / 32]; returns K."""
    what = "[rows, K/2] (two E2M1 codes per byte)" if per_byte == 2 else "[rows, K] (one E4M3 code per byte)"
    require(codes.dim() == 2 and codes.dtype == torch.uint8, f"{op}: {name} must be uint8 {what}")
    require(scales.dim() == 2 and scales.dtype == torch.uint8, f"{op}: {name}_scale must be uint8 [rows, K/32] (E8M0)")
    K = codes.size(1) * per_byte
    require(K > 0 and K % 32 == 0, f"{op}: K={K} must be a positive multiple of 32")
    require(scales.size(0) == codes.size(0) and scales.size(1) == K // 32, f"{op}: {name}_scale shape {tuple(scales.shape)} does not match {name} {tuple(codes.shape)}")
    return K


def check_mx_pair(op: str, a: Tensor, a_scale: Tensor, b: Tensor, b_scale: Tensor, per_byte: int) -> None:
    ka = check_mx_operand(op, "a", a, a_scale, per_byte)
    kb = check_mx_operand(op, "b", b, b_scale, per_byte)
    require(ka == kb, f"{op}: a and b disagree on K ({ka} vs {kb})")
    require(a.size(0) > 0 and b.size(0) > 0, f"{op}: empty operand")


def check_mxfp6_pair(op: str, a: Tensor, a_scale: Tensor, b: Tensor, b_scale: Tensor) -> None:
    for name, codes, scales in (("a", a, a_scale), ("b", b, b_scale)):
        require(codes.dim() == 2 and codes.dtype == torch.uint8, f"{op}: {name} must be uint8 [rows, K*3/4] (packed 6-bit codes)")
        require(scales.dim() == 2 and scales.dtype == torch.uint8, f"{op}: {name}_scale must be uint8 [rows, K/32] (E8M0)")
        require(scales.size(1) > 0 and codes.size(1) == scales.size(1) * 24 and scales.size(0) == codes.size(0),
                f"{op}: {name} {tuple(codes.shape)} and {name}_scale {tuple(scales.shape)} disagree (24 code bytes per scale byte)")
    require(a.size(1) == b.size(1), f"{op}: a and b disagree on K")
    require(a.size(0) > 0 and b.size(0) > 0, f"{op}: empty operand")


FP8_DTYPES = (torch.uint8, torch.float8_e4m3fn)


def check_fp8_operands(op: str, a: Tensor, b: Tensor) -> None:
    require(a.dim() == 2 and b.dim() == 2, f"{op}: a and b must be rank 2")
    require(a.dtype in FP8_DTYPES and b.dtype in FP8_DTYPES, f"{op}: a and b must be float8_e4m3fn (or its bytes as uint8)")
    require(a.size(1) == b.size(1), f"{op}: K mismatch, a is {tuple(a.shape)}, b is {tuple(b.shape)} (b is [N, K])")
    require(a.size(1) > 0 and a.size(1) % 32 == 0, f"{op}: K={a.size(1)} must be a positive multiple of 32")
    require(a.size(0) > 0 and b.size(0) > 0, f"{op}: empty operand")


def check_quantize_input(op: str, x: Tensor) -> None:
    require(x.dim() == 2, f"{op}: x must be [rows, K]")
    require(x.dtype in (torch.float16, torch.bfloat16, torch.float32), f"{op}: dtype {x.dtype} not supported")
    require(x.size(0) > 0 and x.size(1) > 0 and x.size(1) % 32 == 0, f"{op}: K must be a positive multiple of 32")
