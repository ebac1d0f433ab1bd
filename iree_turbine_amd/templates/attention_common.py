from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class AttentionShape:
    """Problem sizes of an attention kernel."""

    num_query_heads: int
    num_kv_heads: int
    head_size: int
    head_size_kv: int
    batch_size: Optional[int] = None
    # prefill
    query_seq_len: Optional[int] = None
    kv_seq_len: Optional[int] = None
    # decode
    num_seqs: Optional[int] = None
    max_seq_len: Optional[int] = None
    block_size: Optional[int] = None
