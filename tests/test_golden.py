"""The committed vectors of tests/golden/fixtures.json: the oracles still reproduce them (CPU), and the kernels
match them through the C ABI without the oracle in the loop (GPU).  tests/golden/make_fixtures.py wrote them."""

import importlib.util
import json
from pathlib import Path

import numpy as np
import pytest
import torch

from conftest import announce

GOLDEN = Path(__file__).with_name("golden")
FIX = json.loads((GOLDEN / "fixtures.json").read_text())


def _maker():
    spec = importlib.util.spec_from_file_location("make_fixtures", GOLDEN / "make_fixtures.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _check(got: torch.Tensor, want: dict, rtol: float, atol: float):
    g = got.detach().double().cpu()
    assert list(g.shape) == want["shape"]
    flat = g.reshape(-1, g.shape[-1])
    np.testing.assert_allclose(flat[:6, :6].numpy(), np.asarray(want["corner"]), rtol=rtol, atol=atol)
    # whole-tensor sums: the error of a sum of n rounded values grows like sqrt(n) * atol at worst like n * atol
    n = g.numel()
    assert abs(float(g.sum()) - want["sum"]) <= atol * n ** 0.5 * 4 + rtol * want["abs_sum"]
    assert abs(float(g.abs().sum()) - want["abs_sum"]) <= atol * n ** 0.5 * 4 + rtol * want["abs_sum"]


@pytest.mark.parametrize("name", sorted(FIX))
def test_oracle_reproduces_fixtures(name):
    mk = _maker()
    assert mk.CASES[name] == FIX[name]["case"]
    now = mk.compute(name)
    want = FIX[name]["expected"]
    assert now.keys() == want.keys()
    for key in want:
        if isinstance(want[key], dict):
            assert now[key]["shape"] == want[key]["shape"]
            # fp32 matmuls add in an order that depends on the host's core count: allow that much
            corner = np.asarray(want[key]["corner"])
            np.testing.assert_allclose(np.asarray(now[key]["corner"]), corner, rtol=1e-5, atol=1e-6 * np.abs(corner).max())
            assert abs(now[key]["sum"] - want[key]["sum"]) <= 1e-6 * want[key]["abs_sum"]
        else:
            assert now[key] == want[key]


@pytest.mark.gpu
def test_kernels_match_fixtures(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs  # the seeded input generator only; no oracle function is called here

    def case(name):
        announce(f"golden {name}")
        return FIX[name]["case"], FIX[name]["expected"]

    c, e = case("gemm_nt")
    a, b = inputs.gemm_inputs(c["M"], c["N"], c["K"], seed=c["seed"])
    _check(torch.ops.mi355.gemm_nt(a.to(dev), b.to(dev), "float32", -1), e["out"], 1e-2, 1e-2)

    c, e = case("flash_attn")
    q, k, v = [t.to(dev) for t in inputs.attention_inputs(c["B"], c["H"], c["Sq"], c["D"], seed=c["seed"])]
    _check(torch.ops.mi355.flash_attn_fwd(q, k, v, False, 0.0), e["noncausal"], 1e-2, 2e-3)
    _check(torch.ops.mi355.flash_attn_fwd(q, k, v, True, 0.0), e["causal"], 1e-2, 2e-3)

    c, e = case("paged_decode")
    q, kc, vc, bt, sl = [t.to(dev) for t in inputs.paged_decode_inputs(**c)]
    _check(torch.ops.mi355.paged_decode_attn(q, kc, vc, bt, sl, 0.0, 2), e["out"], 1e-2, 2e-3)
    _check(torch.ops.mi355.paged_decode_attn_window(q, kc, vc, bt, sl, 0.0, 1, 16), e["window16"], 1e-2, 2e-3)

    c, e = case("paged_prefill")
    kw = {k_: v_ for k_, v_ in c.items() if k_ != "n_new"}
    _, kc, vc, bt, sl = [t.to(dev) for t in inputs.paged_decode_inputs(**kw)]
    qn = torch.randn(c["num_seqs"], c["n_new"], c["num_q_heads"], 128, generator=torch.Generator().manual_seed(c["seed"])).half().to(dev)
    _check(torch.ops.mi355.paged_prefill_attn(qn, kc, vc, bt, sl, 0.0), e["out"], 1e-2, 2e-3)

    c, e = case("mxfp4_gemm")
    args = [t.to(dev) for t in inputs.mxfp4_inputs(c["M"], c["N"], c["K"], seed=c["seed"])]
    _check(torch.ops.mi355.mxfp4_gemm(*args, "float32", -1), e["out"], 1e-5, 1e-5 * max(map(abs, sum(e["out"]["corner"], []))))

    c, e = case("mxfp8_gemm")
    args = [t.to(dev) for t in inputs.mxfp8_inputs(c["M"], c["N"], c["K"], seed=c["seed"])]
    scale = e["out"]["abs_sum"] / (c["M"] * c["N"])
    _check(torch.ops.mi355.mxfp8_gemm(*args, "float32", -1), e["out"], 5e-4, 5e-3 * scale)

    c, e = case("mxfp4_quantize")
    x = (torch.randn(c["rows"], c["K"], generator=torch.Generator().manual_seed(c["seed"])) * 3).half().to(dev)
    codes, scales = torch.ops.mi355.mxfp4_quantize(x)
    assert codes.cpu().tolist() == e["codes"] and scales.cpu().tolist() == e["scales"]

    c, e = case("mxfp8_quantize")
    x = (torch.randn(c["rows"], c["K"], generator=torch.Generator().manual_seed(c["seed"])) * 3).half().to(dev)
    codes, scales = torch.ops.mi355.mxfp8_quantize(x)
    assert codes.cpu().tolist() == e["codes"] and scales.cpu().tolist() == e["scales"]

    c, e = case("mxfp6_gemm")
    args = [t.to(dev) for t in inputs.mxfp6_inputs(c["M"], c["N"], c["K"], seed=c["seed"])]
    for fmt in ("e2m3", "e3m2"):
        scale = e[fmt]["abs_sum"] / (c["M"] * c["N"])
        _check(torch.ops.mi355.mxfp6_gemm(*args, fmt, "float32", -1), e[fmt], 5e-4, 5e-3 * scale)

    c, e = case("mxfp6_quantize")
    x = (torch.randn(c["rows"], c["K"], generator=torch.Generator().manual_seed(c["seed"])) * 3).half().to(dev)
    for fmt in ("e2m3", "e3m2"):
        codes, scales = torch.ops.mi355.mxfp6_quantize(x, fmt)
        assert codes.cpu().tolist() == e[fmt + "_codes"] and scales.cpu().tolist() == e[fmt + "_scales"]
