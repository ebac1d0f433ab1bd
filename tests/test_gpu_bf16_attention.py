"""GPU parity of the bf16 instantiations of the attention kernels (prefill, paged prefill, paged decode, KV
append) through the C ABI vs the CPU oracle on the same bf16 values.

bf16 keeps 8 significand bits: the output's own rounding is up to 2^-9 relative, the probabilities are rounded to
bf16 for the second product and the pre-scaled queries are rounded once more, so the comparison is at
atol = rtol = 1.5e-2 (the fp16 contract of 2e-3 is for fp16 outputs).  Exact properties (a constant V, the
permutation of pages) are checked to the output's rounding."""

import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

TOL = 1.5e-2


def _bf(*ts):
    return [t.bfloat16() for t in ts]


def _to(dev, *ts):
    return [t.to(dev) for t in ts]


@pytest.mark.parametrize("variant", [0, 1, 2, 5, 6])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("Sq,Sk", [(128, 128), (1024, 1024), (100, 100), (333, 333), (96, 320), (1, 77)])
def test_prefill_bf16(dev, Sq, Sk, causal, variant):
    import iree_turbine_amd as ita
    from oracle import attention as oa, inputs

    announce(f"flash_attn_fwd bf16 Sq={Sq} Sk={Sk} causal={causal} variant={variant}")
    q, k, v = _bf(*inputs.attention_inputs(2, 3, Sq, 128, seed=5, Sk=Sk))
    qd, kd, vd = _to(dev, q, k, v)
    o = torch.empty_like(qd)
    ita.launch.flash_attn_fwd_out(qd, kd, vd, o, causal, 0.0, variant)
    assert o.dtype == torch.bfloat16
    torch.testing.assert_close(o.float().cpu(), oa.sdpa_ref(q, k, v, is_causal=causal), rtol=TOL, atol=TOL)
    if ita._lib.variants("flash_attn_fwd")[variant] == "d128_bm128_bn64_w4_m16":  # the op's own choice for these sizes
        assert torch.equal(o, torch.ops.mi355.flash_attn_fwd(qd, kd, vd, causal, 0.0))


@pytest.mark.parametrize("causal", [False, True])
def test_prefill_bf16_grouped_heads_and_strided_views(dev, causal):
    """[B, S, H, D] projections viewed as [B, H, S, D], 8 query heads over 2 key/value heads: read in place."""
    import iree_turbine_amd  # noqa: F401
    from oracle import attention as oa

    announce(f"flash_attn_fwd bf16 gqa strided causal={causal}")
    g = torch.Generator().manual_seed(8)
    B, S, H, Hkv = 2, 200, 8, 2
    q = torch.randn(B, S, H, 128, generator=g).bfloat16()
    k = torch.randn(B, S, Hkv, 128, generator=g).bfloat16()
    v = torch.randn(B, S, Hkv, 128, generator=g).bfloat16()
    o = torch.ops.mi355.flash_attn_fwd(q.to(dev).transpose(1, 2), k.to(dev).transpose(1, 2), v.to(dev).transpose(1, 2), causal, 0.0)
    assert o.dtype == torch.bfloat16 and o.shape == (B, H, S, 128)
    rep = H // Hkv
    ref = oa.sdpa_ref(q.transpose(1, 2), k.transpose(1, 2).repeat_interleave(rep, dim=1),
                      v.transpose(1, 2).repeat_interleave(rep, dim=1), is_causal=causal)
    torch.testing.assert_close(o.float().cpu(), ref, rtol=TOL, atol=TOL)


@pytest.mark.parametrize("causal", [False, True])
def test_prefill_bf16_full_size_properties(dev, causal):
    """B2 H32 S4096: with V = 1 every output is the quotient of the same sum of rounded probabilities by itself, 1 to
    bf16's rounding; the launch is repeatable bit for bit; sampled heads match the oracle."""
    import iree_turbine_amd  # noqa: F401
    from oracle import attention as oa, inputs

    announce(f"flash_attn_fwd bf16 full size causal={causal}")
    q, k, v = _bf(*inputs.attention_inputs(2, 32, 4096, 128))
    qd, kd, vd = _to(dev, q, k, v)
    ones = torch.ones_like(vd)
    o1 = torch.ops.mi355.flash_attn_fwd(qd, kd, ones, causal, 0.0)
    assert (o1.float() - 1.0).abs().max().item() <= 2.0 ** -8
    o = torch.ops.mi355.flash_attn_fwd(qd, kd, vd, causal, 0.0)
    assert torch.equal(o, torch.ops.mi355.flash_attn_fwd(qd, kd, vd, causal, 0.0))
    for b, h in ((0, 0), (1, 31)):
        ref = oa.sdpa_ref(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], is_causal=causal)
        torch.testing.assert_close(o[b:b + 1, h:h + 1].float().cpu(), ref, rtol=TOL, atol=TOL)


@pytest.mark.parametrize("splits", [1, 3, 0])
@pytest.mark.parametrize("hq,hkv", [(32, 8), (8, 8), (16, 1)])
@pytest.mark.parametrize("window", [0, 100])
def test_decode_bf16(dev, hq, hkv, splits, window):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce(f"paged decode bf16 hq={hq} hkv={hkv} splits={splits} window={window}")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=5, num_q_heads=hq, num_kv_heads=hkv, min_len=1, max_len=600, seed=6)
    q, kc, vc = _bf(q, kc, vc)
    args = _to(dev, q, kc, vc, bt, sl)
    if window:
        out = torch.ops.mi355.paged_decode_attn_window(*args, 0.0, splits, window)
    else:
        out = torch.ops.mi355.paged_decode_attn(*args, 0.0, splits)
    assert out.dtype == torch.bfloat16
    ref = op.paged_decode_ref(q, kc, vc, bt, sl, window=window)
    torch.testing.assert_close(out.float().cpu(), ref, rtol=TOL, atol=TOL)


def test_decode_bf16_benchmark_shape_is_page_permutation_invariant(dev):
    """64 sequences, 32 / 8 heads, contexts 512-8192: re-permuting the pages (cache and table together) must not
    change a bit; sampled sequences against the oracle."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce("paged decode bf16 benchmark shape")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs()
    q, kc, vc = _bf(q, kc, vc)
    qd, kd, vd, btd, sld = _to(dev, q, kc, vc, bt, sl)
    out = torch.ops.mi355.paged_decode_attn(qd, kd, vd, btd, sld, 0.0, 0)
    perm = torch.randperm(kc.shape[0], generator=torch.Generator().manual_seed(1)).to(dev)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(perm.numel(), device=dev)
    out2 = torch.ops.mi355.paged_decode_attn(qd, kd[perm], vd[perm], inv[btd.long()].int(), sld, 0.0, 0)
    assert torch.equal(out, out2)
    rows = [0, 17, 63]
    ref = op.paged_decode_ref(q[rows], kc, vc, bt[rows], sl[rows])
    torch.testing.assert_close(out[rows].float().cpu(), ref, rtol=TOL, atol=TOL)


def test_append_then_paged_prefill_bf16(dev):
    """The bf16 serving sequence: append a chunk of new tokens to the paged cache, then attend causally over it."""
    import iree_turbine_amd  # noqa: F401
    from oracle import paged_decode as op

    announce("kv append + paged prefill bf16")
    g = torch.Generator().manual_seed(12)
    S, n_new, Hq, Hkv, page = 3, 96, 8, 2, 16
    prefix = torch.tensor([0, 40, 300], dtype=torch.int32)
    lens = prefix + n_new
    n_pg = (lens + page - 1) // page
    P = int(n_pg.sum()) + 2
    perm = torch.randperm(P, generator=g)
    bt = torch.zeros((S, int(n_pg.max())), dtype=torch.int32)
    off = 0
    for s in range(S):
        n = int(n_pg[s])
        bt[s, :n] = perm[off:off + n].int()
        off += n
    kc = torch.randn(P, page, Hkv, 128, generator=g).bfloat16()
    vc = torch.randn(P, page, Hkv, 128, generator=g).bfloat16()
    kn = torch.randn(S, n_new, Hkv, 128, generator=g).bfloat16()
    vn = torch.randn(S, n_new, Hkv, 128, generator=g).bfloat16()
    q = torch.randn(S, n_new, Hq, 128, generator=g).bfloat16()
    kr, vr = op.kv_cache_append_ref(kn, vn, kc, vc, bt, prefix)
    kd, vd = kc.to(dev), vc.to(dev)
    torch.ops.mi355.kv_cache_append(kn.to(dev), vn.to(dev), kd, vd, bt.to(dev), prefix.to(dev))
    assert torch.equal(kd.cpu(), kr) and torch.equal(vd.cpu(), vr)
    out = torch.ops.mi355.paged_prefill_attn(q.to(dev), kd, vd, bt.to(dev), lens.to(dev), 0.0)
    assert out.dtype == torch.bfloat16
    torch.testing.assert_close(out.float().cpu(), op.paged_prefill_ref(q, kr, vr, bt, lens), rtol=TOL, atol=TOL)


def test_mixed_formats_are_rejected(dev):
    import iree_turbine_amd  # noqa: F401

    q16 = torch.zeros(1, 1, 16, 128, dtype=torch.float16, device=dev)
    qbf = torch.zeros(1, 1, 16, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.flash_attn_fwd(qbf, q16, q16, False, 0.0)
    kc16 = torch.zeros(2, 16, 1, 128, dtype=torch.float16, device=dev)
    bt = torch.zeros(1, 2, dtype=torch.int32, device=dev)
    sl = torch.ones(1, dtype=torch.int32, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.paged_decode_attn(qbf[0, :, 0], kc16, kc16, bt, sl, 0.0, 1)
    with pytest.raises(ValueError):
        torch.ops.mi355.paged_decode_phase0(qbf[0, :, 0], kc16, kc16, bt, sl, 0.0, 2)


def test_decode_bf16_two_phases(dev):
    """Phase 0 on bf16 operands, phase 1 into a bf16 result: bit-identical to the one-call form with as many splits."""
    import iree_turbine_amd as ita
    from oracle import inputs, paged_decode as op

    announce("paged decode bf16 two phases")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=4, min_len=30, max_len=900, seed=2)
    q, kc, vc = _bf(q, kc, vc)
    qd, kd, vd, btd, sld = _to(dev, q, kc, vc, bt, sl)
    pacc, pml = torch.ops.mi355.paged_decode_phase0(qd, kd, vd, btd, sld, 0.0, 4)
    out = torch.empty_like(qd)
    ita.launch.paged_decode_phase1_out(pacc, pml, out)
    assert torch.equal(out, torch.ops.mi355.paged_decode_attn(qd, kd, vd, btd, sld, 0.0, 4))
    torch.testing.assert_close(out.float().cpu(), op.paged_decode_ref(q, kc, vc, bt, sl), rtol=TOL, atol=TOL)
