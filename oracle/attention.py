"""Attention oracle (prefill).  Test infrastructure only (see oracle/__init__.py)."""

from __future__ import annotations

import math

import torch


def causal_mask(sq: int, sk: int) -> torch.Tensor:
    """Additive mask, -inf above the diagonal; lower-right aligned when sq != sk.  For sq == sk this
    is `torch.triu(full(-inf), diagonal=1)` of tests/dynamo/llama_test.py:285-290."""
    m = torch.full((sq, sk), float("-inf"))
    return torch.triu(m, diagonal=1 + (sk - sq))


def sdpa_ref(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, is_causal: bool = False, scale: float | None = None) -> torch.Tensor:
    """softmax(scale . Q K^T + mask) V in fp32, the explicit formula of
    tests/dynamo/llama_test.py:176-180 (scores / sqrt(d), + mask, fp32 softmax, @ values)."""
    qf, kf, vf = (t.detach().cpu().float() for t in (q, k, v))
    if scale is None:
        scale = 1.0 / math.sqrt(qf.shape[-1])
    s = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    if is_causal:
        s = s + causal_mask(qf.shape[-2], kf.shape[-2])
    p = torch.softmax(s, dim=-1)
    return torch.matmul(p, vf)


def sdpa_torch(q, k, v, is_causal=False, scale=None) -> torch.Tensor:
    """torch's own SDPA in fp32 (the library routine the numerical contract names as the oracle)."""
    qf, kf, vf = (t.detach().cpu().float() for t in (q, k, v))
    return torch.nn.functional.scaled_dot_product_attention(qf, kf, vf, is_causal=is_causal, scale=scale)


def sdpa_online(q, k, v, is_causal=False, scale=None, block_n: int = 64) -> torch.Tensor:
    """The online-softmax recurrence of the TK fused attention
    (tests/kernel/fused_attention_test.py:43-76), restated with base e and the 1/sqrt(d) scale:
    running max, running sum rescaled by exp(old_max - new_max), accumulator rescaled likewise, P cast
    to fp16 before the second contraction, final multiply by 1/sum."""
    qf, kf, vf = (t.detach().cpu().float() for t in (q, k, v))
    sq, sk, d = qf.shape[-2], kf.shape[-2], qf.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    lead = qf.shape[:-2]
    m = torch.full((*lead, sq, 1), float("-inf"))
    l = torch.zeros((*lead, sq, 1))
    acc = torch.zeros((*lead, sq, vf.shape[-1]))
    mask = causal_mask(sq, sk) if is_causal else None
    for j in range(0, sk, block_n):
        s = torch.matmul(qf, kf[..., j:j + block_n, :].transpose(-1, -2)) * scale
        if mask is not None:
            s = s + mask[:, j:j + block_n]
        m_new = torch.maximum(m, s.max(dim=-1, keepdim=True).values)
        m_use = torch.where(torch.isinf(m_new), torch.zeros_like(m_new), m_new)
        alpha = torch.exp(m - m_use)
        p = torch.exp(s - m_use)
        l = l * alpha + p.sum(dim=-1, keepdim=True)
        acc = acc * alpha + torch.matmul(p.half().float(), vf[..., j:j + block_n, :])
        m = m_new
    return acc / l
