from __future__ import annotations

import math

from .. import launch
from ..lang import sym
from ..launchable import Launchable
from .attention_common import AttentionShape

BLOCK_M, BLOCK_N = sym.BLOCK_M, sym.BLOCK_N


def _make_entry(is_causal: bool, scale: float | None):
    def entry(hp, q, k, v, o):
        squeeze = q.dim() == 3  # [B*H, S, D] convention
        if squeeze:
            q, k, v, o4 = q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0), o.unsqueeze(0)
        else:
            o4 = o
        launch.flash_attn_fwd_out(q, k, v, o4, is_causal, scale if scale is not None else 1.0 / math.sqrt(q.shape[-1]))

    return entry


def get_vanilla_attention_kernel(shape: AttentionShape, mfma_variant=None, dynamic_dims: bool = False,
                                 is_causal: bool = False, scale: float | None = None):
    """O = softmax(scale . Q K^T [causal]) V, fp32 online softmax.  Call as kernel(q, k, v, o) with
    q, o [B, H, S_q, D] (or [B*H, S_q, D]) and k, v [B, H, S_kv, D], all f16 (or all bf16); o is written in place.

    The recurrence is the fused attention of tests/kernel/fused_attention_test.py:25-77 (running max,
    rescaled running sum and accumulator, P cast to f16 before the second contraction) with the
    1/sqrt(d) scale and base-2 exponent folded together.  Returns (kernel, hyperparams)."""
    if shape.head_size != 128 or shape.head_size_kv != 128:
        raise ValueError(f"get_vanilla_attention_kernel: only head size 128 is built, got {shape.head_size}/{shape.head_size_kv}")
    if shape.num_query_heads != shape.num_kv_heads:
        raise ValueError("get_vanilla_attention_kernel: prefill kernel expects as many kv heads as query heads")
    hyperparams = {BLOCK_M: 128, BLOCK_N: 64}
    kernel = Launchable("flash_attn_fwd_causal" if is_causal else "flash_attn_fwd", _make_entry(is_causal, scale),
                        num_outputs=1, description="flash-attention forward, D=128 (hand-written gfx950 MFMA kernel)")
    return kernel, hyperparams
