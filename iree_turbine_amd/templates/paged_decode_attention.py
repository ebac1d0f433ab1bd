from __future__ import annotations

import math

from .. import launch
from ..lang import sym
from ..launchable import Launchable
from .attention_common import AttentionShape

NUM_KV_SPLITS = sym.U
PAGE_SIZE = sym.BLOCK_SIZE


def paged_decode_attention_shape(num_query_heads: int, num_kv_heads: int, head_size: int, head_size_kv: int,
                                 block_size: int, num_seqs: int, max_seq_len: int | None = None) -> AttentionShape:
    return AttentionShape(num_query_heads=num_query_heads, num_kv_heads=num_kv_heads, head_size=head_size,
                          head_size_kv=head_size_kv, block_size=block_size, num_seqs=num_seqs, max_seq_len=max_seq_len)


def get_paged_decode_attention_kernels(shape: AttentionShape, mfma_variant=None, num_kv_splits: int = 8,
                                       k_shape=None, v_shape=None, block_table_shape=None, scale: float | None = None):
    """Two-phase paged GQA decode attention.

    phase 0: kernel(q, k_cache, v_cache, block_table, seq_lens, part_acc, part_ml)
             q [S, Hq, 128] and caches [P, page, Hkv, 128] f16 (or all bf16); block_table i32 [S, max_pages];
             seq_lens i32 [S]; part_acc f32 [S, Hq, U, 128]; part_ml f32 [S, Hq, U, 2] (outputs)
    phase 1: kernel(part_acc, part_ml, out) with out [S, Hq, 128] f16 or bf16 (output)
    Returns (phase_0, phase_1, hyperparams_0, hyperparams_1).  GQA semantics as repeat_kv,
    tests/dynamo/llama_test.py:82-91."""
    if shape.head_size != 128 or shape.head_size_kv != 128:
        raise ValueError("get_paged_decode_attention_kernels: only head size 128 is built")
    if shape.block_size not in (16, 32, 64, 128, 256):
        raise ValueError(f"get_paged_decode_attention_kernels: pages of 16, 32, 64, 128 or 256 tokens are built, got {shape.block_size}")
    if shape.num_query_heads % shape.num_kv_heads or shape.num_query_heads // shape.num_kv_heads not in (1, 2, 4, 8, 16):
        raise ValueError("get_paged_decode_attention_kernels: q heads per kv head must be 1, 2, 4, 8 or 16")
    if not 1 <= num_kv_splits <= 1024:
        raise ValueError("get_paged_decode_attention_kernels: num_kv_splits must be in [1, 1024]")
    for name, s in (("k_shape", k_shape), ("v_shape", v_shape)):
        if s is not None and tuple(s[1:]) != (shape.block_size, shape.num_kv_heads, 128):
            raise ValueError(f"get_paged_decode_attention_kernels: {name} must be [num_pages, {shape.block_size}, {shape.num_kv_heads}, 128], got {tuple(s)}")

    def phase0(hp, q, k_cache, v_cache, block_table, seq_lens, part_acc, part_ml):
        if part_acc.shape[2] != hp[NUM_KV_SPLITS]:
            raise ValueError(f"phase 0 was built for {hp[NUM_KV_SPLITS]} kv splits, part_acc has {part_acc.shape[2]}")
        launch.paged_decode_phase0_out(q, k_cache, v_cache, block_table, seq_lens, part_acc, part_ml,
                                       scale if scale is not None else 1.0 / math.sqrt(q.shape[-1]))

    def phase1(hp, part_acc, part_ml, out):
        launch.paged_decode_phase1_out(part_acc, part_ml, out)

    hp0 = {NUM_KV_SPLITS: num_kv_splits, PAGE_SIZE: shape.block_size}
    hp1 = {NUM_KV_SPLITS: num_kv_splits}
    return (Launchable("paged_decode_phase0", phase0, num_outputs=2, description="paged GQA decode, split-K phase 0"),
            Launchable("paged_decode_phase1", phase1, num_outputs=1, description="paged GQA decode, split-K merge"),
            hp0, hp1)
