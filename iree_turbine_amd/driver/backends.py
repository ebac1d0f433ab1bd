"""Backends of the driver: how a parsed signature becomes a callable on device tensors.

`mi355` routes the operation to this library's kernels (the role `iree_boo_experimental` plays in the
reference's table, iree/turbine/kernel/boo/driver/driver.py:575-587); `torch` is the eager PyTorch module
(hipBLASLt / SDPA on this device).  A signature the kernels do not cover raises UnsupportedSignature:
the driver reports the row as "N.A." rather than silently running something else.
"""

from __future__ import annotations

from typing import Callable

import torch

from .signatures import AtenSignature, GEMMSignature, OpSignature


class UnsupportedSignature(ValueError):
    pass


class CountingCallable:
    """A callable plus the number of device kernels one call launches (filled in by the first call)."""

    def __init__(self, fn: Callable, name: str):
        self.fn = fn
        self.name = name
        self.dispatches_per_call: int | None = None

    def __call__(self, *args):
        return self.fn(*args)


def _nt_operand(t: torch.Tensor, stored_transposed: bool, counter: list[int]) -> torch.Tensor:
    """The [rows, K] K-contiguous form of a GEMM operand; a copy kernel is counted when one is needed."""
    m = t if stored_transposed else t.t()
    if not m.is_contiguous():
        counter[0] += 1
        m = m.contiguous()
    return m


def _mi355_gemm(sig: GEMMSignature) -> Callable:
    if sig.dtype not in (torch.float16, torch.bfloat16):
        raise UnsupportedSignature(f"{sig.func_name}: the MFMA GEMM takes fp16 or bf16 operands, not {sig.dtype}")
    own = str(sig.dtype).removeprefix("torch.")

    def run(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        n = [1]
        # kernel contract: A[M, K] and B[N, K], both K-contiguous.  A is stored [K, M] under transA;
        # B is stored [N, K] under transB (the native layout) and [K, N] otherwise.
        a_mk = a.t() if sig.transpose_a else a
        if not a_mk.is_contiguous():
            n[0] += 1
            a_mk = a_mk.contiguous()
        b_nk = _nt_operand(b, sig.transpose_b, n)
        out = torch.ops.mi355.gemm_nt(a_mk, b_nk, own, -1)
        run.dispatches = n[0]
        return out

    return run


def _mi355_aten(sig: AtenSignature) -> Callable:
    kwargs = sig.concrete_kwargs()
    types = [t for (_, t, _) in sig.get_non_concrete_args()]
    half_like = {"c10::Half": "float16", "c10::BFloat16": "bfloat16"}
    if sig.name == "aten::mm" and len(set(types)) == 1 and types[0] in half_like:
        own = half_like[types[0]]

        def run(a, b):
            n = [1]
            if not a.is_contiguous():
                n[0] += 1
                a = a.contiguous()
            out = torch.ops.mi355.gemm_nt(a, _nt_operand(b, False, n), own, -1)
            run.dispatches = n[0]
            return out
        return run
    if len(set(types)) != 1 or types[0] not in half_like:
        raise UnsupportedSignature(f"{sig.name}: the kernels take fp16 or bf16 tensors of one dtype, got {types}")
    if sig.name == "aten::scaled_dot_product_attention":
        if kwargs.get("attn_mask") is not None or float(kwargs.get("dropout_p", 0.0) or 0.0) != 0.0:
            raise UnsupportedSignature(f"{sig.name}: attention masks and dropout are not covered")
        if kwargs.get("enable_gqa"):
            raise UnsupportedSignature(f"{sig.name}: enable_gqa is not covered by the prefill kernel")
        dims = [d for (d, _, _) in sig.get_non_concrete_args()]
        if len(dims) != 3 or any(len(d) != 4 for d in dims) or dims[0][3] != 128:
            raise UnsupportedSignature(f"{sig.name}: the prefill kernel covers [B, H, S, 128] tensors, got {dims}")
        causal = bool(kwargs.get("is_causal", False))
        if causal and dims[0][2] != dims[1][2]:
            # aten's mask is aligned to the upper-left corner, the kernel's to the lower-right one
            raise UnsupportedSignature(f"{sig.name}: is_causal with Sq={dims[0][2]} != Sk={dims[1][2]} is not covered "
                                       "(the kernel's causal mask is aligned to the last key)")
        scale = kwargs.get("scale")
        scale = 0.0 if scale is None else float(scale)

        def run(q, k, v):
            n = [1]
            ts = []
            for t in (q, k, v):
                if not t.is_contiguous():
                    n[0] += 1
                    t = t.contiguous()
                ts.append(t)
            out = torch.ops.mi355.flash_attn_fwd(*ts, causal, scale)
            run.dispatches = n[0]
            return out
        return run
    raise UnsupportedSignature(f"{sig.name}: no MI355X kernel for this op")


def mi355_backend(sig: OpSignature) -> CountingCallable:
    import iree_turbine_amd  # noqa: F401  (registers torch.ops.mi355.*; raises if the kernel library is missing)

    if isinstance(sig, GEMMSignature):
        fn = _mi355_gemm(sig)
    elif isinstance(sig, AtenSignature):
        fn = _mi355_aten(sig)
    else:
        raise UnsupportedSignature(f"no MI355X kernel for {type(sig).__name__}")
    cc = CountingCallable(fn, "mi355")

    def call(*args):
        out = fn(*args)
        cc.dispatches_per_call = getattr(fn, "dispatches", 1)
        return out

    cc.fn = call
    return cc


def torch_backend(sig: OpSignature) -> CountingCallable:
    module = sig.get_nn_module()

    def call(*args):
        with torch.no_grad():
            return module(*args)

    return CountingCallable(call, "torch")


DEFAULT_BACKEND = "mi355"
BACKEND_TO_FUNC_GENERATOR: dict[str, Callable[[OpSignature], CountingCallable]] = {
    "mi355": mi355_backend,
    "torch": torch_backend,
}
