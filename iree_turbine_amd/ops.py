"""`torch.ops.mi355.*`: the dense kernels as PyTorch custom ops.

Each op is a `CustomOp` (see op_reg.py): `select` is the shape/dtype contract (and the Meta
kernel), `eager_execute` hands raw device pointers to the C ABI on torch's current stream.
Tensor layouts are the contiguous layouts the reference's launch path enforces
(iree/turbine/runtime/op_reg/eager.py:119-132 makes every input `.contiguous()`).
"""

from __future__ import annotations

import math

import torch
from torch import Tensor

from . import launch
from .contract import PAGE_SIZES, check_mx_operand as _check_mx_operand, check_paged_args as _check_paged_args  # noqa: F401
from . import contract
from .contract import require as _require
from .op_reg import CustomOp, KernelSelection

__all__ = [
    "gemm_nt",
    "flash_attn_fwd",
    "paged_decode_attn",
    "paged_decode_attn_window",
    "kv_cache_append",
    "paged_decode_phase0",
    "paged_decode_phase1",
    "mxfp4_gemm",
    "mxfp4_dequant",
    "mxfp4_quantize",
    "mxfp8_quantize",
    "mxfp6_gemm",
    "mxfp6_quantize",
]

_OUT_DTYPES = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}
_HALF_DTYPES = (torch.float16, torch.bfloat16)  # the attention and GEMM kernels are built for both 16-bit formats


@CustomOp.register
class gemm_nt(CustomOp):
    """C[M,N] = A[M,K] . B[N,K]^T, fp16 or bf16 inputs, fp32 accumulation; out_dtype "float32" or the inputs' own
    ("float16" | "bfloat16").

    The NT form is what `gemmfp16 ... --transB 1` computes in the reference
    (iree/turbine/kernel/boo/op_exports/gemm.py:84-86,228-230) and what `nn.Linear` hands to a
    kernel (tests/kernel/boo/fusion/subgraph_fusion_test.py:100-116)."""

    signature = "gemm_nt(Tensor a, Tensor b, str out_dtype, int variant) -> Tensor"

    def select(self, sel: KernelSelection):
        a, b = sel.arg_tensor(0), sel.arg_tensor(1)
        od = sel.attr_str(2).v
        sel.attr_int(3)
        contract.check_gemm_operands("gemm_nt", a.t, b.t)
        own = str(a.t.dtype).removeprefix("torch.")
        _require(od in ("float32", own), f"gemm_nt: out_dtype must be 'float32' or '{own}' for {own} operands, got {od!r}")
        a.specialize_all_dims()
        b.specialize_all_dims()
        sel.return_new_tensor([a.t.size(0), b.t.size(0)], _OUT_DTYPES[od]).specialize_all_dims()

    def eager_execute(self, a, b, out_dtype, variant):
        c = torch.empty((a.shape[0], b.shape[0]), dtype=_OUT_DTYPES[out_dtype], device=a.device)
        return launch.gemm_nt_out(a, b, c, variant)


def _gemm_nt_setup_context(ctx, inputs, output):
    a, b, _, _ = inputs
    ctx.save_for_backward(a, b)


def _gemm_nt_backward(ctx, grad):
    """For C = A . B^T: dA = dC . B and dB = dC^T . A (the formulas of GEMMBackwardA / GEMMBackwardB,
    iree/turbine/kernel/boo/op_exports/gemm.py:232-269, for the NT layout), each one launch of the same kernel
    on operands re-laid K-contiguous; gradients come back in the operands' dtype."""
    a, b = ctx.saved_tensors
    g = grad.to(a.dtype)
    own = str(a.dtype).removeprefix("torch.")
    grad_a = grad_b = None
    if ctx.needs_input_grad[0]:
        grad_a = torch.ops.mi355.gemm_nt(g.contiguous(), b.t().contiguous(), own, -1)      # [M,N] . [K,N]^T
    if ctx.needs_input_grad[1]:
        grad_b = torch.ops.mi355.gemm_nt(g.t().contiguous(), a.t().contiguous(), own, -1)  # [N,M] . [K,M]^T
    return grad_a, grad_b, None, None


torch.library.register_autograd("mi355::gemm_nt", _gemm_nt_backward, setup_context=_gemm_nt_setup_context)


@CustomOp.register
class flash_attn_fwd(CustomOp):
    """softmax(scale . Q K^T [+ causal mask]) V for q [B,H,Sq,128], k/v [B,Hkv,Sk,128] fp16, H % Hkv == 0
    (query head h reads K/V head h // (H // Hkv), as `enable_gqa=True` does).

    Argument order of aten.scaled_dot_product_attention(q, k, v, None, 0.0, is_causal, scale=) -- the
    canonical form the reference rewrites SDPA variants to (iree/turbine/kernel/boo/fusion/replacement.py:275-284).
    scale <= 0 selects 1/sqrt(D).  One difference in meaning: with Sq != Sk the causal mask is aligned to the LAST
    key (query i sees keys <= i + Sk - Sq, the chunked-prefill convention), where aten aligns it to the first
    (keys <= i); for Sq == Sk the two are the same mask.  The torch.compile pass and the driver backend therefore
    route a causal call to this op only when Sq == Sk.
    The result is laid out like `torch.empty_like(q)`: a transposed [B, S, H, D] view in gives one out."""

    signature = "flash_attn_fwd(Tensor q, Tensor k, Tensor v, bool is_causal, float scale) -> Tensor"

    def select(self, sel: KernelSelection):
        q, k, v = sel.arg_tensor(0), sel.arg_tensor(1), sel.arg_tensor(2)
        sel.attr_bool(3)
        sel.attr_float(4)
        contract.check_attention_operands("flash_attn_fwd", q.t, k.t, v.t)
        for d in (q, k, v):
            d.specialize_dims(1, 3)
        sel.return_tensor(_like_q(q.t, "meta"))

    def eager_execute(self, q, k, v, is_causal, scale):
        return launch.flash_attn_fwd_out(q, k, v, _like_q(q, q.device), is_causal, scale)


def _like_q(q: Tensor, device) -> Tensor:
    """An output with q's dimension order in memory, densely packed (what `empty_like` gives a dense q)."""
    order = sorted(range(4), key=lambda i: (q.stride(i), -i), reverse=True) if q.size(3) > 1 and q.stride(3) == 1 else [0, 1, 2, 3]
    if order[-1] != 3 or any(q.stride(i) == 0 and q.size(i) > 1 for i in range(4)):
        order = [0, 1, 2, 3]
    inv = [order.index(i) for i in range(4)]
    return torch.empty([q.size(i) for i in order], dtype=q.dtype, device=device).permute(inv)


def default_num_kv_splits(seq_lens_max: int, num_seqs: int, num_kv_heads: int) -> int:
    """Splits so that there are about 1500 workgroups (three rounds of the 512 that are resident at once: measured
    best on ragged batches of 16 to 64 sequences, where the kernel walks the sequences longest first), but of at
    least 512 tokens each and at most 32 per sequence: with one to eight sequences every further split costs more
    in partial results and their merge than it gains (1 sequence of 32768 tokens: 37 us with 16-32 splits, 50 with
    64; 8 sequences of 512-4096: 23 us with 4, 28 with 15)."""
    pages = max(1, (seq_lens_max + 15) // 16)
    want = max(1, round(1536 / max(1, num_seqs * num_kv_heads)))
    return int(max(1, min(want, pages // 32 if pages >= 32 else 1, 32)))


@CustomOp.register
class paged_decode_attn(CustomOp):
    """One-token-per-sequence GQA attention over a paged fp16 KV cache (both phases).

    q [S, Hq, 128]; k_cache, v_cache [P, page, Hkv, 128]; block_table int32 [S, max_pages];
    seq_lens int32 [S]; returns [S, Hq, 128] fp16.  num_kv_splits <= 0 picks a default from
    the table width.  scale <= 0 selects 1/sqrt(D).  GQA semantics (q head h reads kv head
    h // (Hq/Hkv)) follow repeat_kv in tests/dynamo/llama_test.py:82-91."""

    signature = "paged_decode_attn(Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_table, Tensor seq_lens, float scale, int num_kv_splits) -> Tensor"

    def select(self, sel: KernelSelection):
        q, kc, vc, bt, sl = (sel.arg_tensor(i) for i in range(5))
        sel.attr_float(5)
        sel.attr_int(6)
        _check_paged_args("paged_decode_attn", q.t, kc.t, vc.t, bt.t, sl.t, bf16_ok=True)
        q.specialize_dims(1, 2)
        kc.specialize_dims(1, 2, 3)
        vc.specialize_dims(1, 2, 3)
        sel.return_new_tensor(list(q.t.shape), q.t.dtype)

    def eager_execute(self, q, k_cache, v_cache, block_table, seq_lens, scale, num_kv_splits):
        if num_kv_splits <= 0:
            num_kv_splits = default_num_kv_splits(block_table.shape[1] * k_cache.shape[1], q.shape[0], k_cache.shape[2])
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        return launch.paged_decode_attn_out(q, k_cache, v_cache, block_table, seq_lens, out, scale, num_kv_splits)


@CustomOp.register
class paged_decode_attn_window(CustomOp):
    """paged_decode_attn restricted to the last `window` cached tokens of every sequence (window == 0: all)."""

    signature = "paged_decode_attn_window(Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_table, Tensor seq_lens, float scale, int num_kv_splits, int window) -> Tensor"

    def select(self, sel: KernelSelection):
        q, kc, vc, bt, sl = (sel.arg_tensor(i) for i in range(5))
        sel.attr_float(5)
        sel.attr_int(6)
        w = sel.attr_int(7).v
        _check_paged_args("paged_decode_attn_window", q.t, kc.t, vc.t, bt.t, sl.t, bf16_ok=True)
        _require(w >= 0, "paged_decode_attn_window: window must be >= 0")
        q.specialize_dims(1, 2)
        kc.specialize_dims(1, 2, 3)
        vc.specialize_dims(1, 2, 3)
        sel.return_new_tensor(list(q.t.shape), q.t.dtype)

    def eager_execute(self, q, k_cache, v_cache, block_table, seq_lens, scale, num_kv_splits, window):
        if num_kv_splits <= 0:
            span = window if window > 0 else block_table.shape[1] * k_cache.shape[1]
            num_kv_splits = default_num_kv_splits(span, q.shape[0], k_cache.shape[2])
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        return launch.paged_decode_attn_out(q, k_cache, v_cache, block_table, seq_lens, out, scale, num_kv_splits, window=window)


@CustomOp.register
class kv_cache_append(CustomOp):
    """In-place paged form of `cache[:bsz, start_pos : start_pos + n_new] = x` (tests/dynamo/llama_test.py:165-166)
    with one start position per sequence: k_new, v_new [S, n_new, Hkv, 128] (fp16 or bf16) go to positions
    start_pos[s] .. start_pos[s] + n_new - 1 of k_cache, v_cache [P, page, Hkv, 128] through block_table [S, max_pages]."""

    signature = "kv_cache_append(Tensor k_new, Tensor v_new, Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor block_table, Tensor start_pos) -> ()"

    def select(self, sel: KernelSelection):
        kn, vn, kc, vc, bt, sp = (sel.arg_tensor(i) for i in range(6))
        contract.check_kv_append("kv_cache_append", kn.t, vn.t, kc.t, vc.t, bt.t, sp.t)

    def eager_execute(self, k_new, v_new, k_cache, v_cache, block_table, start_pos):
        launch.kv_cache_append(k_new, v_new, k_cache, v_cache, block_table, start_pos)
        return None


@CustomOp.register
class paged_prefill_attn(CustomOp):
    """Causal attention of the n_new latest tokens of every sequence over its paged KV cache (chunked / prefix
    prefill): q [S, n_new, Hq, 128], caches [P, page, Hkv, 128], block_table int32 [S, max_pages], seq_lens int32 [S]
    counting the new tokens, whose K/V are in the cache already (kv_cache_append).  Query t sees positions
    j <= seq_lens[s] - n_new + t: the mask of tests/dynamo/llama_test.py:285-290 shifted by the cached prefix."""

    signature = "paged_prefill_attn(Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_table, Tensor seq_lens, float scale) -> Tensor"

    def select(self, sel: KernelSelection):
        q, kc, vc, bt, sl = (sel.arg_tensor(i) for i in range(5))
        sel.attr_float(5)
        contract.check_paged_prefill("paged_prefill_attn", q.t, kc.t, vc.t, bt.t, sl.t)
        q.specialize_dims(2, 3)
        sel.return_new_tensor(list(q.t.shape), q.t.dtype)

    def eager_execute(self, q, k_cache, v_cache, block_table, seq_lens, scale):
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        return launch.paged_prefill_attn_out(q, k_cache, v_cache, block_table, seq_lens, out, scale)


@CustomOp.register
class paged_decode_phase0(CustomOp):
    """Phase 0 of the split-K decode: per (seq, q head, split) an unnormalised fp32 partial
    output [S, Hq, splits, 128] and its (max in log2 units, sum) [S, Hq, splits, 2]."""

    signature = "paged_decode_phase0(Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_table, Tensor seq_lens, float scale, int num_kv_splits) -> (Tensor, Tensor)"

    def select(self, sel: KernelSelection):
        q, kc, vc, bt, sl = (sel.arg_tensor(i) for i in range(5))
        sel.attr_float(5)
        ns = sel.attr_int(6).v
        _check_paged_args("paged_decode_phase0", q.t, kc.t, vc.t, bt.t, sl.t, bf16_ok=True)
        _require(1 <= ns <= 1024, "paged_decode_phase0: num_kv_splits must be in [1, 1024]")
        S, Hq, D = q.t.shape
        sel.return_new_tensor([S, Hq, ns, D], torch.float32)
        sel.return_new_tensor([S, Hq, ns, 2], torch.float32)

    def eager_execute(self, q, k_cache, v_cache, block_table, seq_lens, scale, num_kv_splits):
        S, Hq, D = q.shape
        pacc = torch.empty((S, Hq, num_kv_splits, D), dtype=torch.float32, device=q.device)
        pml = torch.empty((S, Hq, num_kv_splits, 2), dtype=torch.float32, device=q.device)
        launch.paged_decode_phase0_out(q, k_cache, v_cache, block_table, seq_lens, pacc, pml, scale)
        return pacc, pml


@CustomOp.register
class paged_decode_phase1(CustomOp):
    """Phase 1 of the split-K decode: merges the partials of phase 0 into [S, Hq, 128] fp16 (a bf16 result comes
    from `launch.paged_decode_phase1_out` with a bf16 `out`, or from the one-call `paged_decode_attn`)."""

    signature = "paged_decode_phase1(Tensor part_acc, Tensor part_ml) -> Tensor"

    def select(self, sel: KernelSelection):
        pa, pm = sel.arg_tensor(0), sel.arg_tensor(1)
        _require(pa.t.dim() == 4 and pa.t.dtype == torch.float32 and pa.t.size(3) == 128, "paged_decode_phase1: part_acc must be fp32 [S, Hq, splits, 128]")
        _require(pm.t.dtype == torch.float32 and tuple(pm.t.shape) == (*pa.t.shape[:3], 2), "paged_decode_phase1: part_ml must be fp32 [S, Hq, splits, 2]")
        sel.return_new_tensor([pa.t.size(0), pa.t.size(1), 128], torch.float16)

    def eager_execute(self, part_acc, part_ml):
        S, Hq, _, D = part_acc.shape
        out = torch.empty((S, Hq, D), dtype=torch.float16, device=part_acc.device)
        return launch.paged_decode_phase1_out(part_acc, part_ml, out)


@CustomOp.register
class mxfp4_gemm(CustomOp):
    """C[M,N] = dq(A) . dq(B)^T for OCP MXFP4 operands (see include/turbine_mi355.h for the format);
    out_dtype "bfloat16" | "float32"."""

    signature = "mxfp4_gemm(Tensor a, Tensor a_scale, Tensor b, Tensor b_scale, str out_dtype, int variant) -> Tensor"

    def select(self, sel: KernelSelection):
        a, asc, b, bsc = (sel.arg_tensor(i) for i in range(4))
        od = sel.attr_str(4).v
        sel.attr_int(5)
        contract.check_mx_pair("mxfp4_gemm", a.t, asc.t, b.t, bsc.t, per_byte=2)
        _require(od in ("bfloat16", "float32"), f"mxfp4_gemm: out_dtype must be 'bfloat16' or 'float32', got {od!r}")
        for d in (a, asc, b, bsc):
            d.specialize_all_dims()
        sel.return_new_tensor([a.t.size(0), b.t.size(0)], _OUT_DTYPES[od]).specialize_all_dims()

    def eager_execute(self, a, a_scale, b, b_scale, out_dtype, variant):
        c = torch.empty((a.shape[0], b.shape[0]), dtype=_OUT_DTYPES[out_dtype], device=a.device)
        return launch.mxfp4_gemm_out(a, a_scale, b, b_scale, c, variant)


@CustomOp.register
class mxfp8_gemm(CustomOp):
    """C[M,N] = dq(A) . dq(B)^T for OCP MXFP8 operands: E4M3 codes uint8 [rows, K] (torch.float8_e4m3fn viewed as
    uint8), E8M0 scales uint8 [rows, K/32]; out_dtype "bfloat16" | "float32"."""

    signature = "mxfp8_gemm(Tensor a, Tensor a_scale, Tensor b, Tensor b_scale, str out_dtype, int variant) -> Tensor"

    def select(self, sel: KernelSelection):
        a, asc, b, bsc = (sel.arg_tensor(i) for i in range(4))
        od = sel.attr_str(4).v
        sel.attr_int(5)
        contract.check_mx_pair("mxfp8_gemm", a.t, asc.t, b.t, bsc.t, per_byte=1)
        _require(od in ("bfloat16", "float32"), f"mxfp8_gemm: out_dtype must be 'bfloat16' or 'float32', got {od!r}")
        for d in (a, asc, b, bsc):
            d.specialize_all_dims()
        sel.return_new_tensor([a.t.size(0), b.t.size(0)], _OUT_DTYPES[od]).specialize_all_dims()

    def eager_execute(self, a, a_scale, b, b_scale, out_dtype, variant):
        c = torch.empty((a.shape[0], b.shape[0]), dtype=_OUT_DTYPES[out_dtype], device=a.device)
        return launch.mxfp8_gemm_out(a, a_scale, b, b_scale, c, variant)


@CustomOp.register
class mxfp6_gemm(CustomOp):
    """C[M,N] = dq(A) . dq(B)^T for OCP MXFP6 operands: 6-bit codes packed as a little-endian bit stream, uint8
    [rows, K*3/4] (element k at bits [6k, 6k+6) of its row), E8M0 scales uint8 [rows, K/32]; element_format
    "e2m3" (the reference's f6E2M3FN, iree/turbine/kernel/_support/dtype.py:118) | "e3m2"; out_dtype "bfloat16" |
    "float32"."""

    signature = "mxfp6_gemm(Tensor a, Tensor a_scale, Tensor b, Tensor b_scale, str element_format, str out_dtype, int variant) -> Tensor"

    def select(self, sel: KernelSelection):
        a, asc, b, bsc = (sel.arg_tensor(i) for i in range(4))
        fmt = sel.attr_str(4).v
        od = sel.attr_str(5).v
        sel.attr_int(6)
        contract.check_mxfp6_pair("mxfp6_gemm", a.t, asc.t, b.t, bsc.t)
        _require(fmt in launch.FP6_FORMATS, f"mxfp6_gemm: element_format must be 'e2m3' or 'e3m2', got {fmt!r}")
        _require(od in ("bfloat16", "float32"), f"mxfp6_gemm: out_dtype must be 'bfloat16' or 'float32', got {od!r}")
        for d in (a, asc, b, bsc):
            d.specialize_all_dims()
        sel.return_new_tensor([a.t.size(0), b.t.size(0)], _OUT_DTYPES[od]).specialize_all_dims()

    def eager_execute(self, a, a_scale, b, b_scale, element_format, out_dtype, variant):
        c = torch.empty((a.shape[0], b.shape[0]), dtype=_OUT_DTYPES[out_dtype], device=a.device)
        return launch.mxfp6_gemm_out(a, a_scale, b, b_scale, c, element_format, variant)


@CustomOp.register
class fp8_gemm(CustomOp):
    """C[M,N] = alpha . A . B^T for E4M3 operands: a [M, K], b [N, K] as torch.float8_e4m3fn or the same bytes as
    uint8; out_dtype "bfloat16" | "float32".  alpha = the product of the per-tensor scales used when quantising."""

    signature = "fp8_gemm(Tensor a, Tensor b, float alpha, str out_dtype, int variant) -> Tensor"

    def select(self, sel: KernelSelection):
        a, b = sel.arg_tensor(0), sel.arg_tensor(1)
        sel.attr_float(2)
        od = sel.attr_str(3).v
        sel.attr_int(4)
        contract.check_fp8_operands("fp8_gemm", a.t, b.t)
        _require(od in ("bfloat16", "float32"), f"fp8_gemm: out_dtype must be 'bfloat16' or 'float32', got {od!r}")
        a.specialize_all_dims()
        b.specialize_all_dims()
        sel.return_new_tensor([a.t.size(0), b.t.size(0)], _OUT_DTYPES[od]).specialize_all_dims()

    def eager_execute(self, a, b, alpha, out_dtype, variant):
        c = torch.empty((a.shape[0], b.shape[0]), dtype=_OUT_DTYPES[out_dtype], device=a.device)
        return launch.fp8_gemm_out(a, b, c, alpha, variant)


@CustomOp.register
class mxfp4_dequant(CustomOp):
    """fp32 [rows, K] = E2M1(code) * 2^(scale - 127), computed on the device."""

    signature = "mxfp4_dequant(Tensor codes, Tensor scales) -> Tensor"

    def select(self, sel: KernelSelection):
        c, s = sel.arg_tensor(0), sel.arg_tensor(1)
        _check_mx_operand("mxfp4_dequant", "codes", c.t, s.t)
        _require(c.t.size(0) > 0, "mxfp4_dequant: empty operand")
        sel.return_new_tensor([c.t.size(0), c.t.size(1) * 2], torch.float32)

    def eager_execute(self, codes, scales):
        out = torch.empty((codes.shape[0], codes.shape[1] * 2), dtype=torch.float32, device=codes.device)
        return launch.mxfp4_dequant_out(codes, scales, out)


@CustomOp.register
class mxfp4_quantize(CustomOp):
    """(codes uint8 [rows, K/2], scales uint8 [rows, K/32]) of x [rows, K] (fp16, bf16 or fp32): the OCP MX
    conversion -- block exponent floor(log2(max|x|)) - 2, round to nearest E2M1, ties to the even code."""

    signature = "mxfp4_quantize(Tensor x) -> (Tensor, Tensor)"

    def select(self, sel: KernelSelection):
        x = sel.arg_tensor(0)
        contract.check_quantize_input("mxfp4_quantize", x.t)
        sel.return_new_tensor([x.t.size(0), x.t.size(1) // 2], torch.uint8)
        sel.return_new_tensor([x.t.size(0), x.t.size(1) // 32], torch.uint8)

    def eager_execute(self, x):
        codes = torch.empty((x.shape[0], x.shape[1] // 2), dtype=torch.uint8, device=x.device)
        scales = torch.empty((x.shape[0], x.shape[1] // 32), dtype=torch.uint8, device=x.device)
        return launch.mxfp4_quantize_out(x, codes, scales)


@CustomOp.register
class mxfp6_quantize(CustomOp):
    """(codes uint8 [rows, K*3/4], scales uint8 [rows, K/32]) of x [rows, K] (fp16, bf16 or fp32): the OCP MX
    conversion to 6-bit elements, element_format "e2m3" | "e3m2" -- block exponent floor(log2(max|x|)) - emax
    (2 / 4), round to nearest, ties to the even code, saturating at 7.5 / 28; codes packed as mxfp6_gemm reads them."""

    signature = "mxfp6_quantize(Tensor x, str element_format) -> (Tensor, Tensor)"

    def select(self, sel: KernelSelection):
        x = sel.arg_tensor(0)
        fmt = sel.attr_str(1).v
        contract.check_quantize_input("mxfp6_quantize", x.t)
        _require(fmt in launch.FP6_FORMATS, f"mxfp6_quantize: element_format must be 'e2m3' or 'e3m2', got {fmt!r}")
        sel.return_new_tensor([x.t.size(0), x.t.size(1) // 4 * 3], torch.uint8)
        sel.return_new_tensor([x.t.size(0), x.t.size(1) // 32], torch.uint8)

    def eager_execute(self, x, element_format):
        codes = torch.empty((x.shape[0], x.shape[1] // 4 * 3), dtype=torch.uint8, device=x.device)
        scales = torch.empty((x.shape[0], x.shape[1] // 32), dtype=torch.uint8, device=x.device)
        return launch.mxfp6_quantize_out(x, codes, scales, element_format)


@CustomOp.register
class mxfp8_quantize(CustomOp):
    """(codes uint8 [rows, K], scales uint8 [rows, K/32]) of x [rows, K] (fp16, bf16 or fp32): the OCP MX
    conversion to E4M3 elements -- block exponent floor(log2(max|x|)) - 8, round to nearest, ties to the even
    code, saturating at 448.  The codes view as torch.float8_e4m3fn."""

    signature = "mxfp8_quantize(Tensor x) -> (Tensor, Tensor)"

    def select(self, sel: KernelSelection):
        x = sel.arg_tensor(0)
        contract.check_quantize_input("mxfp8_quantize", x.t)
        sel.return_new_tensor([x.t.size(0), x.t.size(1)], torch.uint8)
        sel.return_new_tensor([x.t.size(0), x.t.size(1) // 32], torch.uint8)

    def eager_execute(self, x):
        codes = torch.empty((x.shape[0], x.shape[1]), dtype=torch.uint8, device=x.device)
        scales = torch.empty((x.shape[0], x.shape[1] // 32), dtype=torch.uint8, device=x.device)
        return launch.mxfp8_quantize_out(x, codes, scales)
