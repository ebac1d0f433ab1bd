"""Writes tests/golden/fixtures.json: for a few small seeded cases of every kernel family, a corner of the
oracle's result and two whole-tensor sums.  Data only -- the inputs are regenerated from the seeds by
oracle/inputs.py.  Run from the repository root:  python tests/golden/make_fixtures.py

The reference's kernels for this path are not in its checkout and nothing of it was imported or run; the
vectors come from the CPU oracles (each pinned independently in tests/test_oracle_*.py) and freeze their
behaviour, so that a later change to an oracle or to the input generator cannot go unnoticed, and give the
GPU tests a target that does not execute the oracle."""

import json
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import attention as oa, inputs, mxfp4 as o4, mxfp6 as o6, mxfp8 as o8, paged_decode as op  # noqa: E402

CASES = {
    "gemm_nt": dict(M=96, N=80, K=160, seed=3),
    "flash_attn": dict(B=1, H=2, Sq=70, D=128, seed=4),
    "paged_decode": dict(num_seqs=4, num_q_heads=8, num_kv_heads=2, min_len=3, max_len=150, seed=5),
    "paged_prefill": dict(num_seqs=3, num_q_heads=8, num_kv_heads=2, min_len=30, max_len=150, seed=5, n_new=20),
    "mxfp4_gemm": dict(M=64, N=96, K=256, seed=6),
    "mxfp8_gemm": dict(M=64, N=96, K=256, seed=6),
    "mxfp4_quantize": dict(rows=8, K=64, seed=7),
    "mxfp8_quantize": dict(rows=8, K=64, seed=7),
    "mxfp6_gemm": dict(M=64, N=96, K=256, seed=6),
    "mxfp6_quantize": dict(rows=8, K=64, seed=7),
}


def summarise(t: torch.Tensor) -> dict:
    t = t.detach().double()
    flat = t.reshape(-1, t.shape[-1])
    return {"shape": list(t.shape), "corner": flat[:6, :6].tolist(), "sum": float(t.sum()), "abs_sum": float(t.abs().sum())}


def compute(name: str) -> dict:
    c = CASES[name]
    if name == "gemm_nt":
        a, b = inputs.gemm_inputs(c["M"], c["N"], c["K"], seed=c["seed"])
        return {"out": summarise(a.float() @ b.float().t())}
    if name == "flash_attn":
        q, k, v = inputs.attention_inputs(c["B"], c["H"], c["Sq"], c["D"], seed=c["seed"])
        return {"noncausal": summarise(oa.sdpa_ref(q, k, v, is_causal=False)), "causal": summarise(oa.sdpa_ref(q, k, v, is_causal=True))}
    if name in ("paged_decode", "paged_prefill"):
        kw = {k: v for k, v in c.items() if k != "n_new"}
        q, kc, vc, bt, sl = inputs.paged_decode_inputs(**kw)
        if name == "paged_decode":
            return {"out": summarise(op.paged_decode_ref(q, kc, vc, bt, sl)), "window16": summarise(op.paged_decode_ref(q, kc, vc, bt, sl, window=16))}
        qn = torch.randn(c["num_seqs"], c["n_new"], c["num_q_heads"], 128, generator=torch.Generator().manual_seed(c["seed"])).half()
        return {"out": summarise(op.paged_prefill_ref(qn, kc, vc, bt, sl))}
    if name == "mxfp4_gemm":
        return {"out": summarise(o4.mxfp4_gemm_ref(*inputs.mxfp4_inputs(c["M"], c["N"], c["K"], seed=c["seed"])))}
    if name == "mxfp8_gemm":
        return {"out": summarise(o8.mxfp8_gemm_ref(*inputs.mxfp8_inputs(c["M"], c["N"], c["K"], seed=c["seed"])))}
    if name == "mxfp4_quantize":
        x = (torch.randn(c["rows"], c["K"], generator=torch.Generator().manual_seed(c["seed"])) * 3).half()
        codes, scales = o4.mxfp4_quantize_ref(x)
        return {"codes": np.asarray(codes).astype(int).tolist(), "scales": np.asarray(scales).astype(int).tolist()}
    if name == "mxfp8_quantize":
        x = (torch.randn(c["rows"], c["K"], generator=torch.Generator().manual_seed(c["seed"])) * 3).half()
        codes, scales = o8.mxfp8_quantize_ref(x)
        return {"codes": np.asarray(codes).astype(int).tolist(), "scales": np.asarray(scales).astype(int).tolist()}
    if name == "mxfp6_gemm":
        args = inputs.mxfp6_inputs(c["M"], c["N"], c["K"], seed=c["seed"])
        return {"e2m3": summarise(o6.mxfp6_gemm_ref(*args, "e2m3")), "e3m2": summarise(o6.mxfp6_gemm_ref(*args, "e3m2"))}
    if name == "mxfp6_quantize":
        x = (torch.randn(c["rows"], c["K"], generator=torch.Generator().manual_seed(c["seed"])) * 3).half()
        out = {}
        for fmt in ("e2m3", "e3m2"):
            codes, scales = o6.mxfp6_quantize_ref(x, fmt)
            out[fmt + "_codes"] = np.asarray(codes).astype(int).tolist()
            out[fmt + "_scales"] = np.asarray(scales).astype(int).tolist()
        return out
    raise KeyError(name)


if __name__ == "__main__":
    out = {name: {"case": CASES[name], "expected": compute(name)} for name in CASES}
    path = Path(__file__).with_name("fixtures.json")
    path.write_text(json.dumps(out, indent=1) + "\n")
    print(f"wrote {path} ({path.stat().st_size} bytes)")
