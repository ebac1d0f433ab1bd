"""Paged GQA decode-attention oracle.  Test infrastructure only (see oracle/__init__.py)."""

from __future__ import annotations

import math

import torch


def gather_kv(cache: torch.Tensor, block_table_row: torch.Tensor, length: int) -> torch.Tensor:
    """[length, Hkv, D]: tokens of one sequence, page by page through its block-table row."""
    page = cache.shape[1]
    n_pages = (length + page - 1) // page
    ids = block_table_row[:n_pages].long()
    return cache[ids].reshape(n_pages * page, cache.shape[2], cache.shape[3])[:length]


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[len, Hkv, D] -> [len, Hkv * n_rep, D]; q head h reads kv head h // n_rep
    (tests/dynamo/llama_test.py:82-91)."""
    if n_rep == 1:
        return x
    ln, hkv, d = x.shape
    return x[:, :, None, :].expand(ln, hkv, n_rep, d).reshape(ln, hkv * n_rep, d)


def paged_decode_ref(q, k_cache, v_cache, block_table, seq_lens, scale: float | None = None, window: int = 0) -> torch.Tensor:
    """out[s, h] = softmax(q[s, h] . K_s^T * scale) V_s over the first seq_lens[s] cached tokens,
    fp32 softmax (llama_test.py:160-181 with one query token).  window > 0: only the last `window` of them."""
    qf = q.detach().cpu().float()
    kc, vc = k_cache.detach().cpu().float(), v_cache.detach().cpu().float()
    bt, sl = block_table.detach().cpu(), seq_lens.detach().cpu()
    S, Hq, D = qf.shape
    n_rep = Hq // kc.shape[2]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    out = torch.zeros((S, Hq, D), dtype=torch.float32)
    for s in range(S):
        ln = int(sl[s])
        if ln == 0:
            continue
        lo = max(0, ln - window) if window > 0 else 0
        ks = repeat_kv(gather_kv(kc, bt[s], ln)[lo:], n_rep)  # [len - lo, Hq, D]
        vs = repeat_kv(gather_kv(vc, bt[s], ln)[lo:], n_rep)
        scores = torch.einsum("hd,lhd->hl", qf[s], ks) * scale
        p = torch.softmax(scores, dim=-1)
        out[s] = torch.einsum("hl,lhd->hd", p, vs)
    return out


def kv_cache_append_ref(k_new, v_new, k_cache, v_cache, block_table, start_pos):
    """Copies of the caches with cache[:, start_pos[s] : start_pos[s] + n_new] = new for every sequence,
    addressed through the block table (llama_test.py:165-166); positions without a valid table entry are
    skipped."""
    kc, vc = k_cache.detach().cpu().clone(), v_cache.detach().cpu().clone()
    page = kc.shape[1]
    bt = block_table.detach().cpu()
    for s in range(k_new.shape[0]):
        for t in range(k_new.shape[1]):
            pos = int(start_pos[s]) + t
            if pos < 0 or pos // page >= bt.shape[1]:
                continue
            pg = int(bt[s, pos // page])
            if pg < 0 or pg >= kc.shape[0]:
                continue
            kc[pg, pos % page] = k_new[s, t].cpu()
            vc[pg, pos % page] = v_new[s, t].cpu()
    return kc, vc


def paged_prefill_ref(q, k_cache, v_cache, block_table, seq_lens, scale: float | None = None) -> torch.Tensor:
    """out[s, t, h] = softmax over the cached positions j <= seq_lens[s] - n_new + t of q[s, t, h] . K_s[j] * scale,
    times V_s: the attention of tests/dynamo/llama_test.py:160-181 with the mask of :285-290 (query t of the
    new chunk sees the cached prefix and the chunk up to itself), K/V gathered through the block table.
    q [S, n_new, Hq, D]; a query with no visible position gives zeros."""
    qf = q.detach().cpu().float()
    kc, vc = k_cache.detach().cpu().float(), v_cache.detach().cpu().float()
    bt, sl = block_table.detach().cpu(), seq_lens.detach().cpu()
    S, T, Hq, D = qf.shape
    n_rep = Hq // kc.shape[2]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    out = torch.zeros((S, T, Hq, D), dtype=torch.float32)
    for s in range(S):
        ln = max(0, min(int(sl[s]), bt.shape[1] * kc.shape[1]))
        if ln == 0:
            continue
        ks = repeat_kv(gather_kv(kc, bt[s], ln), n_rep)  # [ln, Hq, D]
        vs = repeat_kv(gather_kv(vc, bt[s], ln), n_rep)
        scores = torch.einsum("thd,lhd->thl", qf[s], ks) * scale
        pos = torch.arange(ln)[None, :]
        last = (ln - T + torch.arange(T))[:, None]  # last visible position of query t
        visible = pos <= last  # [T, ln]
        scores = scores.masked_fill(~visible[:, None, :], float("-inf"))
        p = torch.softmax(scores, dim=-1)
        p = torch.where(visible.any(dim=1)[:, None, None], p, torch.zeros_like(p))  # rows with nothing visible
        out[s] = torch.einsum("thl,lhd->thd", p, vs)
    return out
