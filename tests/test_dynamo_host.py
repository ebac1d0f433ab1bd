"""Host-side tests of the torch.compile routing pass: which ATen nodes are handed to the MI355X kernels.

The graphs are traced from CPU tensors (no GPU here), so the pass is told to accept any device; nothing is
executed -- the assertions are on graph structure.  The pass plays the role of the reference's fusion schema +
SDPA canonicalisation (iree/turbine/kernel/boo/fusion/schema.py:106-135, fusion/replacement.py:239-284), and the
cases follow tests/kernel/boo/fusion/subgraph_fusion_test.py (linear layers) and
tests/kernel/boo/fusion/replacement_test.py (SDPA variants, declined when auxiliary outputs are used)."""

import operator

import pytest
import torch
import torch.nn.functional as F
from torch.fx.experimental.proxy_tensor import make_fx

ANY = lambda dev: True


def _targets(gm):
    return [n.target for n in gm.graph.nodes if n.op == "call_function"]


def _trace(f, *args):
    return make_fx(f)(*args)


def _h(*shape):
    return torch.randn(*shape).half()


def test_linear_layers_become_gemm_nt_without_copies():
    from iree_turbine_amd import dynamo

    x, w, b = _h(64, 256), _h(512, 256), _h(512)
    gm = _trace(lambda x, w, b: F.linear(x, w, b) + x @ w.t(), x, w, b)
    counts = dynamo.substitute_kernels(gm, device_ok=ANY)
    assert counts == {"mm": 1, "addmm": 1, "sdpa": 0}
    ts = _targets(gm)
    assert torch.ops.aten.mm.default not in ts and torch.ops.aten.addmm.default not in ts
    gemms = [n for n in gm.graph.nodes if n.target is torch.ops.mi355.gemm_nt.default]
    assert len(gemms) == 2
    names = {n.name: n for n in gm.graph.nodes if n.op == "placeholder"}
    for g in gemms:  # the [N, K] weight itself is the B operand: the transposes died
        assert g.args[0] is names["x_1"] and g.args[1] is names["w_1"] and g.args[2] == "float16"
    assert torch.ops.aten.t.default not in ts


def test_mm_with_untransposed_rhs_gets_a_transpose():
    from iree_turbine_amd import dynamo

    gm = _trace(lambda a, b: a @ b, _h(32, 64), _h(64, 48))
    assert dynamo.substitute_kernels(gm, device_ok=ANY)["mm"] == 1
    g = next(n for n in gm.graph.nodes if n.target is torch.ops.mi355.gemm_nt.default)
    assert g.args[1].target is torch.ops.aten.t.default  # b^T is [N, K]; the launcher packs it


def test_bf16_linear_layers_keep_their_dtype():
    from iree_turbine_amd import dynamo

    x, w, b = _h(64, 256).bfloat16(), _h(512, 256).bfloat16(), _h(512).bfloat16()
    gm = _trace(lambda x, w, b: F.linear(x, w, b) + x @ w.t(), x, w, b)
    assert dynamo.substitute_kernels(gm, device_ok=ANY) == {"mm": 1, "addmm": 1, "sdpa": 0}
    gemms = [n for n in gm.graph.nodes if n.target is torch.ops.mi355.gemm_nt.default]
    assert len(gemms) == 2 and all(g.args[2] == "bfloat16" for g in gemms)


@pytest.mark.parametrize("what", ["fp32", "fp64", "addmm_beta", "empty"])
def test_unsupported_matmuls_are_left_alone(what):
    from iree_turbine_amd import dynamo

    if what == "fp32":
        gm = _trace(lambda a, b: a @ b, torch.randn(8, 8), torch.randn(8, 8))
    elif what == "fp64":
        gm = _trace(lambda a, b: a @ b, torch.randn(8, 8).double(), torch.randn(8, 8).double())
    elif what == "addmm_beta":
        gm = _trace(lambda c, a, b: torch.addmm(c, a, b, beta=0.5), _h(8, 8), _h(8, 8), _h(8, 8))
    else:
        gm = _trace(lambda a, b: a @ b, _h(0, 8), _h(8, 8))
    before = _targets(gm)
    assert sum(dynamo.substitute_kernels(gm, device_ok=ANY).values()) == 0
    assert _targets(gm) == before


def test_default_device_filter_declines_cpu_graphs():
    from iree_turbine_amd import dynamo

    gm = _trace(lambda a, b: a @ b.t(), _h(8, 8), _h(8, 8))
    assert sum(dynamo.substitute_kernels(gm).values()) == 0


def _sdpa_fn(causal=False, mask=False, dropout=0.0, scale=None):
    def attend(q, k, v, m):
        o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                           attn_mask=m, dropout_p=dropout, is_causal=causal, scale=scale)
        return o.transpose(1, 2).reshape(q.shape[0], q.shape[1], -1)

    if mask:
        return lambda q, k, v, m: attend(q, k, v, m)
    return lambda q, k, v: attend(q, k, v, None)


@pytest.mark.parametrize("causal", [False, True])
def test_sdpa_is_rewritten_to_the_single_output_kernel(causal):
    from iree_turbine_amd import dynamo

    q, k, v = _h(2, 96, 4, 128), _h(2, 96, 4, 128), _h(2, 96, 4, 128)
    gm = _trace(_sdpa_fn(causal=causal, scale=0.25), q, k, v)
    assert dynamo.substitute_kernels(gm, device_ok=ANY)["sdpa"] == 1
    ts = _targets(gm)
    assert operator.getitem not in ts and not any(t in dynamo._SDPA_VARIANTS for t in ts)
    fa = next(n for n in gm.graph.nodes if n.target is torch.ops.mi355.flash_attn_fwd.default)
    assert fa.args[3] is causal and fa.args[4] == 0.25
    # q is a transposed [B, S, H, D] view and so is the kernel's result: no layout fix-up was needed
    assert torch.ops.aten.clone.default not in ts
    assert fa.meta["val"].stride() == q.transpose(1, 2).stride()


@pytest.mark.parametrize("what", ["mask", "head_dim", "fp32", "causal_unequal_lengths"])
def test_unsupported_sdpa_is_left_alone(what):
    from iree_turbine_amd import dynamo

    if what == "causal_unequal_lengths":  # aten masks keys > i, the kernel keys > i + Sk - Sq
        gm = _trace(_sdpa_fn(causal=True), _h(1, 32, 2, 128), _h(1, 96, 2, 128), _h(1, 96, 2, 128))
    elif what == "mask":
        gm = _trace(_sdpa_fn(mask=True), _h(1, 32, 2, 128), _h(1, 32, 2, 128), _h(1, 32, 2, 128), _h(32, 32))
    elif what == "head_dim":
        gm = _trace(_sdpa_fn(), _h(1, 32, 2, 64), _h(1, 32, 2, 64), _h(1, 32, 2, 64))
    else:
        gm = _trace(_sdpa_fn(), torch.randn(1, 32, 2, 128), torch.randn(1, 32, 2, 128), torch.randn(1, 32, 2, 128))
    before = _targets(gm)
    assert dynamo.substitute_kernels(gm, device_ok=ANY)["sdpa"] == 0
    assert _targets(gm) == before


def test_sdpa_with_used_auxiliary_output_is_left_alone():
    """The log-sum-exp feeds the backward graph in training: the multi-output node must survive
    (fusion/replacement.py:262-266 declines the same way)."""
    from iree_turbine_amd import dynamo

    variant = next(iter(dynamo._SDPA_VARIANTS))
    name = dynamo._SDPA_VARIANTS[variant]
    if name != "_scaled_dot_product_flash_attention_for_cpu":
        variant = torch.ops.aten._scaled_dot_product_flash_attention_for_cpu.default

    def f(q, k, v):
        out, lse = variant(q, k, v)
        return out, lse

    gm = _trace(f, _h(1, 2, 32, 128), _h(1, 2, 32, 128), _h(1, 2, 32, 128))
    assert dynamo.substitute_kernels(gm, device_ok=ANY)["sdpa"] == 0


def test_sdpa_result_layout_is_reproduced_when_the_variant_differs_from_q():
    """A variant that writes [B, S, H, D] whatever q's layout (the memory-efficient kernel): later nodes were
    traced against those strides, so the pass re-creates them with one packed copy."""
    from iree_turbine_amd import dynamo

    def f(q, k, v):
        return torch.ops.aten._scaled_dot_product_flash_attention_for_cpu.default(q, k, v)[0]

    q = _h(2, 4, 32, 128)
    gm = _trace(f, q, q.clone(), q.clone())
    get0 = next(n for n in gm.graph.nodes if n.target is operator.getitem and n.args[1] == 0)
    get0.meta["val"] = torch.empty(2, 32, 4, 128, dtype=torch.float16, device="meta").transpose(1, 2)
    assert dynamo.substitute_kernels(gm, device_ok=ANY)["sdpa"] == 1
    out = next(n for n in gm.graph.nodes if n.op == "output").args[0]
    assert out.target is torch.ops.aten.permute.default and out.args[1] == [0, 2, 1, 3]
    clone = out.args[0]
    assert clone.target is torch.ops.aten.clone.default and clone.args[0].args[1] == [0, 2, 1, 3]
    assert clone.args[0].args[0].target is torch.ops.mi355.flash_attn_fwd.default


def test_backends_are_registered():
    import iree_turbine_amd.dynamo  # noqa: F401

    names = torch._dynamo.list_backends(exclude_tags=None)
    assert "mi355" in names and "mi355_inductor" not in names
    with pytest.raises(ValueError, match="Triton"):
        iree_turbine_amd.dynamo.backend(nested_backend="inductor")
