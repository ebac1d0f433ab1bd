"""`torch.compile` routing: a backend that substitutes this library's kernels for the ATen ops they cover.

    model = torch.compile(model, backend="mi355")            # registered on import
    model = torch.compile(model, backend=iree_turbine_amd.dynamo.backend(nested_backend=my_compiler_fn))

The role of the reference's `iree_boo_experimental` backend (iree/turbine/dynamo/backends/boo.py:55-126),
whose schema roots offloading at `aten.mm` / `aten.addmm` and the `_scaled_dot_product_*` variants
(iree/turbine/kernel/boo/fusion/schema.py:106-135) and rewrites the multi-output attention variants into the
single-output form when their auxiliary outputs are unused (fusion/replacement.py:239-284).  Here the
substitution is a direct FX rewrite of the ATen graph that AOT-autograd produces:

  aten.mm(x, t(w))            -> mi355.gemm_nt(x, w)                 (w is already [N, K]: no copy)
  aten.mm(x, b)               -> mi355.gemm_nt(x, contiguous(t(b)))
  aten.addmm(bias, x, t(w))   -> mi355.gemm_nt(x, w) + bias           (beta = alpha = 1 only)
  aten._scaled_dot_product_{flash,efficient,flash_for_cpu}_attention(q, k, v, ...)[0]
                              -> mi355.flash_attn_fwd(q, k, v, is_causal, scale)

A node is rewritten only when the kernels cover it (fp16 or bf16 tensors of one dtype on a CUDA device, head dim 128, no mask, no dropout, a causal mask only with Sq == Sk, auxiliary outputs unused -- so training graphs keep PyTorch's attention); everything else is left
for the nested backend.  Layouts: the ops make their operands contiguous themselves, so transposed views
(`q.transpose(1, 2)`) need no graph surgery.
"""

from __future__ import annotations

import operator
import warnings
from typing import Callable

import torch
from torch import fx

aten = torch.ops.aten

_SDPA_VARIANTS = {}
for _name in ("_scaled_dot_product_flash_attention", "_scaled_dot_product_flash_attention_for_cpu",
              "_scaled_dot_product_efficient_attention"):
    if hasattr(aten, _name):
        _SDPA_VARIANTS[getattr(aten, _name).default] = _name


def _val(node):
    return node.meta.get("val") if isinstance(node, fx.Node) else None


_GEMM_DTYPES = (torch.float16, torch.bfloat16)


def _is_half_matrix(node, device_ok, dtype=None) -> bool:
    """A non-empty rank-2 fp16 / bf16 tensor on a device the backend serves (of exactly `dtype` if given)."""
    v = _val(node)
    return (isinstance(v, torch.Tensor) and v.dim() == 2 and v.dtype in _GEMM_DTYPES and (dtype is None or v.dtype == dtype)
            and device_ok(v.device) and v.numel() > 0)


def _transposed_source(node):
    """w if node is t(w) / transpose(w, 0, 1) / permute(w, [1, 0]) of a matrix, else None."""
    if not isinstance(node, fx.Node) or node.op != "call_function":
        return None
    if node.target is aten.t.default:
        return node.args[0]
    if node.target is aten.transpose.int and sorted(d % 2 for d in node.args[1:3]) == [0, 1]:
        return node.args[0]
    if node.target is aten.permute.default and list(node.args[1]) == [1, 0]:
        return node.args[0]
    return None


def _gemm_nt_node(graph: fx.Graph, a, b):
    """Inserts gemm_nt(a, b_nk) for aten.mm(a, b): b_nk is b's [N, K] K-contiguous form."""
    src = _transposed_source(b)
    v = _val(src)
    if src is not None and isinstance(v, torch.Tensor) and v.is_contiguous():
        b_nk = src
    else:
        b_nk = graph.call_function(aten.t.default, (b,))
    own = str(_val(a).dtype).removeprefix("torch.")
    return graph.call_function(torch.ops.mi355.gemm_nt.default, (a, b_nk, own, -1))


def _rewrite_mm(node: fx.Node, device_ok) -> bool:
    a, b = node.args[:2]
    if not _is_half_matrix(a, device_ok):
        return False
    dt = _val(a).dtype
    if not (_is_half_matrix(b, device_ok, dt) and _is_half_matrix(node, device_ok, dt)):
        return False
    with node.graph.inserting_before(node):
        new = _gemm_nt_node(node.graph, a, b)
    new.meta = dict(node.meta)
    node.replace_all_uses_with(new)
    node.graph.erase_node(node)
    return True


def _rewrite_addmm(node: fx.Node, device_ok) -> bool:
    bias, a, b = node.args[:3]
    if node.kwargs.get("beta", 1) != 1 or node.kwargs.get("alpha", 1) != 1:
        return False
    bv = _val(bias)
    if not _is_half_matrix(a, device_ok):
        return False
    dt = _val(a).dtype
    if not (_is_half_matrix(b, device_ok, dt) and _is_half_matrix(node, device_ok, dt)):
        return False
    if not (isinstance(bv, torch.Tensor) and bv.dtype == dt and bv.dim() in (1, 2)):
        return False
    with node.graph.inserting_before(node):
        mm = _gemm_nt_node(node.graph, a, b)
        new = node.graph.call_function(aten.add.Tensor, (mm, bias))
    mm.meta = dict(node.meta)
    new.meta = dict(node.meta)
    node.replace_all_uses_with(new)
    node.graph.erase_node(node)
    return True


def _rewrite_sdpa(node: fx.Node, device_ok) -> bool:
    name = _SDPA_VARIANTS[node.target]
    schema = node.target._schema
    bound = {a.name: (node.args[i] if i < len(node.args) else node.kwargs.get(a.name, a.default_value))
             for i, a in enumerate(schema.arguments)}
    q, k, v = bound["query"], bound["key"], bound["value"]
    if bound.get("attn_bias") is not None or bound.get("attn_mask") is not None:
        return False
    if float(bound.get("dropout_p", 0.0) or 0.0) != 0.0:
        return False
    vals = [_val(t) for t in (q, k, v)]
    if not all(isinstance(t, torch.Tensor) and t.dim() == 4 and t.dtype in _GEMM_DTYPES and device_ok(t.device) for t in vals):
        return False
    if len({t.dtype for t in vals}) != 1:
        return False
    qv, kv, vv = vals
    if qv.shape[-1] != 128 or kv.shape != vv.shape or qv.shape[0] != kv.shape[0] or kv.shape[-1] != 128:
        return False
    if qv.shape[1] != kv.shape[1]:
        return False
    if min(qv.shape[2], kv.shape[2]) == 0 or qv.numel() == 0:
        return False
    if bool(bound.get("is_causal", False)) and qv.shape[2] != kv.shape[2]:
        # aten aligns the causal mask to the upper-left corner (query i sees keys <= i); the kernel aligns it to the
        # lower-right one (the last query sees every key).  The two agree only for Sq == Sk.
        return False
    getitems = [u for u in node.users if u.op == "call_function" and u.target is operator.getitem]
    if len(getitems) != len(node.users):
        return False
    out_user = None
    for u in getitems:
        if u.args[1] == 0:
            out_user = u
        elif len(u.users) > 0:
            return False  # log-sum-exp / RNG state used downstream (a training graph): keep PyTorch's kernel
    if out_user is None:
        return False
    scale = bound.get("scale")
    want = _val(out_user)
    got = _like(qv)
    restride = None
    if isinstance(want, torch.Tensor) and want.stride() != got.stride():
        # the variant lays its result out differently from q (the efficient kernel always writes [B, S, H, D]):
        # later nodes were traced against those strides, so reproduce them with one packed copy
        restride = sorted(range(4), key=lambda i: (want.stride(i), -i), reverse=True)
        packed = torch.empty([want.size(i) for i in restride], device="meta").permute([restride.index(i) for i in range(4)])
        if packed.stride() != want.stride():
            return False
    with node.graph.inserting_before(node):
        new = node.graph.call_function(torch.ops.mi355.flash_attn_fwd.default,
                                       (q, k, v, bool(bound.get("is_causal", False)), 0.0 if scale is None else float(scale)))
        new.meta = dict(out_user.meta)
        if restride is not None:
            new.meta["val"] = got
            p = node.graph.call_function(aten.permute.default, (new, restride))
            c = node.graph.call_function(aten.clone.default, (p,), {"memory_format": torch.contiguous_format})
            new = node.graph.call_function(aten.permute.default, (c, [restride.index(i) for i in range(4)]))
            new.meta = dict(out_user.meta)
    out_user.replace_all_uses_with(new)
    for u in getitems:
        node.graph.erase_node(u)
    node.graph.erase_node(node)
    return True


def _like(q: torch.Tensor) -> torch.Tensor:
    from .ops import _like_q

    return _like_q(q, "meta")


def substitute_kernels(gm: fx.GraphModule, device_ok: Callable[[torch.device], bool] | None = None) -> dict[str, int]:
    """Rewrites `gm` in place; returns how many nodes of each kind were routed to the MI355X kernels."""
    import iree_turbine_amd  # noqa: F401  (registers torch.ops.mi355.*; raises if the kernel library is missing)

    if device_ok is None:
        device_ok = lambda d: d.type == "cuda"
    counts = {"mm": 0, "addmm": 0, "sdpa": 0}
    for node in list(gm.graph.nodes):
        if node.op != "call_function":
            continue
        if node.target is aten.mm.default:
            counts["mm"] += _rewrite_mm(node, device_ok)
        elif node.target is aten.addmm.default:
            counts["addmm"] += _rewrite_addmm(node, device_ok)
        elif node.target in _SDPA_VARIANTS:
            counts["sdpa"] += _rewrite_sdpa(node, device_ok)
    if any(counts.values()):
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()
    return counts


LAST_SUBSTITUTIONS: dict[str, int] = {}


def backend(*, nested_backend="eager"):
    """A `torch.compile` backend: kernels substituted in the forward ATen graph, the rest compiled by
    `nested_backend` (any registered backend name or compiler function)."""
    from functorch.compile import make_boxed_func
    from torch._dynamo.backends.common import aot_autograd

    if nested_backend == "inductor":
        # inductor compiles the rest of the graph into Triton kernels; this library ships hand-written HIP only
        raise ValueError("nested_backend='inductor' is not supported: it would generate Triton kernels for the remaining "
                         "graph; use 'eager' (the default) or a compiler function of your own")
    if nested_backend != "eager" and not callable(nested_backend):
        warnings.warn(f"nested_backend {nested_backend!r} is not known to preserve the substituted ops")
    nested_fn = torch._dynamo.lookup_backend(nested_backend)

    def compiler_fn(gm: fx.GraphModule, example_inputs):
        LAST_SUBSTITUTIONS.update(substitute_kernels(gm))
        return make_boxed_func(nested_fn(gm, example_inputs))

    return aot_autograd(fw_compiler=compiler_fn)


def _register() -> None:
    from torch._dynamo.backends.registry import register_backend

    try:
        register_backend(name="mi355", compiler_fn=backend())
    except Exception:  # already registered (module re-import)
        pass


_register()
