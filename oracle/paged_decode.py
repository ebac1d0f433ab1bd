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
