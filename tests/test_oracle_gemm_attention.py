"""Pins the GEMM and attention oracles with checks that do not restate their formulas: brute force,
closed forms, a library routine, and invariants chosen so that a dropped term, a wrong sign or a
transposed operand fails at least one of them.  (The reference holds no numeric golden files for
these kernels; its own KATs for the harness arithmetic are restated in test_oracle_numerics.py.)"""

import math

import numpy as np
import pytest
import torch

from oracle import attention as oa, gemm as og, inputs


def test_gemm_ref_vs_bruteforce():
    a, b = inputs.gemm_inputs(13, 9, 21, seed=1)
    bf = og.gemm_nt_bruteforce(a, b)
    np.testing.assert_allclose(og.gemm_nt_ref(a, b).numpy(), bf, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(og.gemm_nt_f64(a, b).numpy(), bf, rtol=1e-12, atol=1e-12)
    # a transposed-operand mistake would change the shape or the values
    assert og.gemm_nt_ref(a, b).shape == (13, 9)


def test_gemm_ref_special_cases():
    b = (torch.randn(24, 32) * 0.5).half()
    assert torch.equal(og.gemm_nt_ref(torch.eye(32).half(), b), b.float().t())  # A = I  =>  C = B^T
    a1 = torch.zeros(8, 64).half()
    a1[2:5, 10:50] = 1
    b1 = torch.ones(6, 64).half()
    exp = torch.zeros(8, 6)
    exp[2:5] = 40
    assert torch.equal(og.gemm_nt_ref(a1, b1), exp)  # block of ones: exact integer sums
    # K-split invariance: summing over two halves of K equals the whole
    a, b = inputs.gemm_inputs(16, 16, 128, seed=2)
    whole = og.gemm_nt_f64(a, b)
    parts = og.gemm_nt_f64(a[:, :64], b[:, :64]) + og.gemm_nt_f64(a[:, 64:], b[:, 64:])
    torch.testing.assert_close(whole, parts, rtol=1e-12, atol=1e-12)


def test_gemm_tiled_restatement_matches():
    a, b = inputs.gemm_inputs(70, 45, 100, seed=3)
    torch.testing.assert_close(og.gemm_nt_tiled(a, b), og.gemm_nt_ref(a, b), rtol=1e-5, atol=1e-5)


def test_input_generator_anchor():
    # first draws of torch.Generator("cpu").manual_seed(10): identical inputs on every box
    g = torch.Generator(device="cpu").manual_seed(10)
    x = torch.randn(3, generator=g)
    np.testing.assert_allclose(x.numpy(), [-0.6013928055763245, -1.0122097730636597, -0.30226925015449524], rtol=0, atol=1e-7)
    a, b = inputs.gemm_inputs(4, 5, 8)
    g = torch.Generator(device="cpu").manual_seed(10)
    a2 = (torch.randn((4, 8), generator=g) * 0.1).half()
    b2 = (torch.randn((5, 8), generator=g) * 0.1).half()
    assert torch.equal(a, a2) and torch.equal(b, b2)  # A drawn before B, in stored [rows, K] shapes


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("sq,sk", [(37, 37), (16, 50), (64, 64)])
def test_sdpa_ref_vs_torch_library(causal, sq, sk):
    if causal and sq != sk:
        pytest.skip("torch's is_causal is upper-left aligned when lengths differ")
    q, k, v = inputs.attention_inputs(2, 3, sq, 32, seed=4, Sk=sk)
    torch.testing.assert_close(oa.sdpa_ref(q, k, v, causal), oa.sdpa_torch(q, k, v, causal), rtol=1e-5, atol=1e-6)


def test_sdpa_ref_bruteforce_single_row():
    q, k, v = inputs.attention_inputs(1, 1, 5, 8, seed=6)
    qn, kn, vn = (t[0, 0].double().numpy() for t in (q, k, v))
    for causal in (False, True):
        out = np.zeros((5, 8))
        for i in range(5):
            n = i + 1 if causal else 5
            w = np.array([math.exp(float(qn[i] @ kn[j]) / math.sqrt(8)) for j in range(n)])
            out[i] = (w[:, None] * vn[:n]).sum(0) / w.sum()
        np.testing.assert_allclose(oa.sdpa_ref(q, k, v, causal)[0, 0].numpy(), out, rtol=1e-5, atol=1e-6)


def test_sdpa_invariants():
    q, k, v = inputs.attention_inputs(1, 2, 48, 16, seed=7)
    ones = torch.ones_like(v)
    torch.testing.assert_close(oa.sdpa_ref(q, k, ones), torch.ones(1, 2, 48, 16), rtol=0, atol=1e-6)  # rows of P sum to 1
    assert torch.equal(oa.sdpa_ref(q, k, v, True)[:, :, 0], v.float()[:, :, 0])  # causal row 0 = V[0]
    z = torch.zeros_like(q)
    pref = v.float().cumsum(2) / torch.arange(1, 49).view(1, 1, 48, 1)
    torch.testing.assert_close(oa.sdpa_ref(z, k, v, True), pref, rtol=1e-5, atol=1e-6)  # Q = 0: prefix means
    perm = torch.randperm(48, generator=torch.Generator().manual_seed(0))
    torch.testing.assert_close(oa.sdpa_ref(q, k[:, :, perm], v[:, :, perm]), oa.sdpa_ref(q, k, v), rtol=1e-5, atol=1e-6)
    # causal mask for unequal lengths is lower-right aligned: last query sees every key
    m = oa.causal_mask(3, 5)
    assert (m[-1] == 0).all() and (m[0] == torch.tensor([0, 0, 0, float("-inf"), float("-inf")])).all()


@pytest.mark.parametrize("causal", [False, True])
def test_online_softmax_restatement(causal):
    q, k, v = inputs.attention_inputs(1, 2, 150, 32, seed=8)
    # differs from the direct formula only by the fp16 rounding of P (as in the TK kernel)
    torch.testing.assert_close(oa.sdpa_online(q, k, v, causal, block_n=64), oa.sdpa_ref(q, k, v, causal), rtol=2e-3, atol=2e-3)
    torch.testing.assert_close(oa.sdpa_online(q, k, v, causal, block_n=32), oa.sdpa_online(q, k, v, causal, block_n=150), rtol=2e-3, atol=2e-3)
