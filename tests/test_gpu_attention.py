"""GPU parity: flash-attention prefill through the C ABI vs the CPU oracle (fp32 SDPA), atol 2e-3."""

import math

import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

ATOL = 2e-3  # the contract tolerance for fp16 attention outputs
RTOL = 1e-2


def _run(dev, B, H, Sq, D, causal, seed=10, Sk=None):
    import iree_turbine_amd  # noqa: F401
    from oracle import attention as oa, inputs

    announce(f"flash_attn_fwd B={B} H={H} Sq={Sq} Sk={Sk} D={D} causal={causal} seed={seed}")
    q, k, v = inputs.attention_inputs(B, H, Sq, D, seed=seed, Sk=Sk)
    o = torch.ops.mi355.flash_attn_fwd(q.to(dev), k.to(dev), v.to(dev), causal, 0.0)
    torch.cuda.synchronize()
    return o.float().cpu(), oa.sdpa_ref(q, k, v, is_causal=causal), (q, k, v)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("S", [128, 256, 1024])
def test_attention_aligned(dev, S, causal):
    o, ref, _ = _run(dev, 2, 4, S, 128, causal)
    torch.testing.assert_close(o, ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("S", [1, 17, 64, 100, 129, 333])
def test_attention_ragged(dev, S, causal):
    o, ref, _ = _run(dev, 1, 3, S, 128, causal)
    torch.testing.assert_close(o, ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("causal", [False, True])
def test_attention_cross_lengths(dev, causal):
    o, ref, _ = _run(dev, 1, 2, 96, 128, causal, Sk=320)
    torch.testing.assert_close(o, ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("Sq,Sk", [(1, 1), (64, 64), (255, 255), (257, 257), (300, 777), (1024, 1024), (700, 100)])
def test_attention_eight_wave_form(dev, Sq, Sk, causal):
    """The 8-wave form (256 queries per workgroup, both wave quartets sharing one copy of every K / V tile): ragged
    and cross lengths, query counts around the 256-query block, Sq > Sk -- against the oracle, and bit-identical to
    the 4-wave form (same per-wave arithmetic, only the tile loads are split differently)."""
    import iree_turbine_amd as ita
    from oracle import attention as oa, inputs

    announce(f"flash_attn_fwd 8 waves Sq={Sq} Sk={Sk} causal={causal}")
    names = ita._lib.variants("flash_attn_fwd")
    v8 = names.index("d128_bm256_bn64_w8_pipelined")
    q, k, v = inputs.attention_inputs(2, 3, Sq, 128, seed=12, Sk=Sk)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    o8, o4 = torch.empty_like(qd), torch.empty_like(qd)
    ita.launch.flash_attn_fwd_out(qd, kd, vd, o8, causal, 0.0, v8)
    ita.launch.flash_attn_fwd_out(qd, kd, vd, o4, causal, 0.0, 0)
    assert torch.equal(o8, o4)
    got = o8.float().cpu()
    if causal and Sq > Sk:
        got, q = got[:, :, Sq - Sk:], q[:, :, Sq - Sk:]  # the first Sq - Sk queries see no key (zeros, checked elsewhere)
    torch.testing.assert_close(got, oa.sdpa_ref(q, k, v, is_causal=causal), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("Sq,Sk", [(1, 1), (17, 17), (64, 64), (100, 100), (255, 255), (257, 257), (300, 777), (1024, 1024), (700, 100),
                                   (96, 320), (2048, 2048)])
def test_attention_16x16x32_forms(dev, Sq, Sk, causal):
    """The forms on 16x16x32 MFMAs (the automatic choice; a lane owns one query of either 16-query group and a quarter of
    a tile's keys, so masks, row sums and the rare rescale are laid out differently from the 32x32x16 forms): ragged and
    cross lengths, lengths around the block sizes, Sq > Sk, several tiles -- against the oracle; the 4- and the 8-wave
    form agree bit for bit (same per-wave arithmetic, only the exponentials sit at other places of the trip), and
    both agree with the 32x32x16 form to the rounding of the output."""
    import iree_turbine_amd as ita
    from oracle import attention as oa, inputs

    announce(f"flash_attn_fwd 16x16x32 forms Sq={Sq} Sk={Sk} causal={causal}")
    names = ita._lib.variants("flash_attn_fwd")
    q, k, v = inputs.attention_inputs(2, 3, Sq, 128, seed=16, Sk=Sk)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    o4, o8, o32 = torch.empty_like(qd), torch.empty_like(qd), torch.empty_like(qd)
    ita.launch.flash_attn_fwd_out(qd, kd, vd, o4, causal, 0.0, names.index("d128_bm128_bn64_w4_m16"))
    ita.launch.flash_attn_fwd_out(qd, kd, vd, o8, causal, 0.0, names.index("d128_bm256_bn64_w8_m16"))
    ita.launch.flash_attn_fwd_out(qd, kd, vd, o32, causal, 0.0, 0)
    assert torch.equal(o4, o8)
    torch.testing.assert_close(o4.float(), o32.float(), rtol=RTOL, atol=ATOL)
    assert torch.equal(o4, torch.ops.mi355.flash_attn_fwd(qd, kd, vd, causal, 0.0))  # what the op runs at these sizes
    got = o4.float().cpu()
    if causal and Sq > Sk:
        assert torch.equal(got[:, :, :Sq - Sk], torch.zeros_like(got[:, :, :Sq - Sk]))  # queries that see no key
        got, q = got[:, :, Sq - Sk:], q[:, :, Sq - Sk:]
    torch.testing.assert_close(got, oa.sdpa_ref(q, k, v, is_causal=causal), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("form", ["d128_bm256_bn64_w8_walk", "d128_bm128_bn64_w4_walk"])
@pytest.mark.parametrize("B,H,Sq,Sk", [(2, 3, 128, 128), (1, 2, 255, 255), (1, 2, 257, 257), (2, 3, 320, 320), (1, 5, 777, 777),
                                       (3, 40, 1024, 1024), (2, 3, 300, 777), (1, 2, 700, 128), (1, 9, 192, 4200)])
def test_attention_persistent_forms(dev, B, H, Sq, Sk, form, causal):
    """The persistent forms (one workgroup per CU slot running its passes back to back, the next pass's rows and first
    tiles requested under the current pass's last tile): passes of even and odd tile counts, ragged lengths, more
    units than workgroup slots (3 x 40 heads), a single workgroup per head -- against the oracle and bit-identical to
    the 4-wave form, whose arithmetic per query they repeat.  The masked form only takes square problems."""
    import iree_turbine_amd as ita
    from oracle import attention as oa, inputs

    announce(f"flash_attn_fwd {form} B={B} H={H} Sq={Sq} Sk={Sk} causal={causal}")
    vw = ita._lib.variants("flash_attn_fwd").index(form)
    q, k, v = inputs.attention_inputs(B, H, Sq, 128, seed=14, Sk=Sk)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    ow, o4 = torch.empty_like(qd), torch.empty_like(qd)
    if causal and Sq != Sk:
        with pytest.raises(ValueError, match="persistent form"):
            ita.launch.flash_attn_fwd_out(qd, kd, vd, ow, causal, 0.0, vw)
        return
    ita.launch.flash_attn_fwd_out(qd, kd, vd, ow, causal, 0.0, vw)
    ita.launch.flash_attn_fwd_out(qd, kd, vd, o4, causal, 0.0, 0)
    assert torch.equal(ow, o4)
    if B * H <= 12:
        torch.testing.assert_close(ow.float().cpu(), oa.sdpa_ref(q, k, v, is_causal=causal), rtol=RTOL, atol=ATOL)


def test_attention_persistent_forms_need_two_tiles(dev):
    """A pass of the persistent forms has at least two key tiles: fewer than 128 keys is refused, nothing is launched."""
    import iree_turbine_amd as ita
    from oracle import inputs

    announce("flash_attn_fwd persistent forms, Sk < 128")
    q, k, v = [t.to(dev) for t in inputs.attention_inputs(1, 2, 100, 128, seed=15)]
    o = torch.full_like(q, 7.0)
    for form in ("d128_bm256_bn64_w8_walk", "d128_bm128_bn64_w4_walk"):
        with pytest.raises(ValueError, match="Sk >= 128"):
            ita.launch.flash_attn_fwd_out(q, k, v, o, False, 0.0, ita._lib.variants("flash_attn_fwd").index(form))
    assert bool((o == 7.0).all())


def test_attention_causal_more_queries_than_keys(dev):
    """Lower-right aligned causal mask with Sq > Sk: query i sees keys j <= i - (Sq - Sk), so the first
    Sq - Sk queries see no key at all.  Those rows are defined as zero (the sum of an empty softmax); every
    other row matches the oracle."""
    import iree_turbine_amd  # noqa: F401
    from oracle import attention as oa, inputs

    B, H, Sq, Sk, D = 1, 2, 300, 100, 128  # the boundary falls inside a wave: rows with and without keys side by side
    announce(f"flash_attn_fwd causal Sq={Sq} > Sk={Sk}")
    q, k, v = inputs.attention_inputs(B, H, Sq, D, seed=11, Sk=Sk)
    o = torch.ops.mi355.flash_attn_fwd(q.to(dev), k.to(dev), v.to(dev), True, 0.0).float().cpu()
    empty = Sq - Sk
    assert torch.equal(o[:, :, :empty], torch.zeros_like(o[:, :, :empty]))
    ref = oa.sdpa_ref(q[:, :, empty:], k, v, is_causal=True)  # the remaining Sk queries against Sk keys: square mask
    torch.testing.assert_close(o[:, :, empty:], ref, rtol=RTOL, atol=ATOL)


def test_attention_invariants(dev):
    import iree_turbine_amd  # noqa: F401

    announce("attention invariants")
    B, H, S, D = 1, 2, 512, 128
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, H, S, D, generator=g).half().to(dev)
    k = torch.randn(B, H, S, D, generator=g).half().to(dev)
    v = torch.randn(B, H, S, D, generator=g).half().to(dev)
    # rows of P sum to one: V = 1 => O = 1
    o = torch.ops.mi355.flash_attn_fwd(q, k, torch.ones_like(v), False, 0.0)
    assert (o.float() - 1).abs().max().item() <= 1e-3
    # causal row 0 sees only key 0
    oc = torch.ops.mi355.flash_attn_fwd(q, k, v, True, 0.0)
    assert torch.equal(oc[:, :, 0], v[:, :, 0])
    # Q = 0: uniform weights => prefix means (causal) / the mean (non-causal) of V
    z = torch.zeros_like(q)
    om = torch.ops.mi355.flash_attn_fwd(z, k, v, False, 0.0).float()
    torch.testing.assert_close(om, v.float().mean(dim=2, keepdim=True).expand_as(om), rtol=1e-2, atol=2e-3)
    op = torch.ops.mi355.flash_attn_fwd(z, k, v, True, 0.0).float()
    pref = v.float().cumsum(dim=2) / torch.arange(1, S + 1, device=dev).view(1, 1, S, 1)
    torch.testing.assert_close(op, pref, rtol=1e-2, atol=2e-3)
    # permuting the keys (with their values) does not change non-causal attention
    perm = torch.randperm(S, generator=g).to(dev)
    o1 = torch.ops.mi355.flash_attn_fwd(q, k, v, False, 0.0).float()
    o2 = torch.ops.mi355.flash_attn_fwd(q, k[:, :, perm], v[:, :, perm], False, 0.0).float()
    torch.testing.assert_close(o1, o2, rtol=1e-2, atol=2e-3)


@pytest.mark.parametrize("causal", [False, True])
def test_attention_full_size(dev, causal):
    """B=2 H=32 S=4096 D=128: two full heads against the oracle, every head against torch's GPU SDPA."""
    import iree_turbine_amd  # noqa: F401
    from oracle import attention as oa, inputs

    announce(f"attention full size causal={causal}")
    q, k, v = inputs.attention_inputs(2, 32, 4096, 128)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    o = torch.ops.mi355.flash_attn_fwd(qd, kd, vd, causal, 0.0)
    for (b, h) in [(0, 0), (1, 31)]:
        ref = oa.sdpa_ref(q[b, h], k[b, h], v[b, h], is_causal=causal)
        torch.testing.assert_close(o[b, h].float().cpu(), ref, rtol=RTOL, atol=ATOL)
    lib = torch.nn.functional.scaled_dot_product_attention(qd.float(), kd.float(), vd.float(), is_causal=causal)
    torch.testing.assert_close(o.float(), lib, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("causal", [False, True])
def test_attention_full_size_repeatable(dev, causal):
    """Every kernel variant gives bit-identical output on repeated launches at full size, and the variants
    agree with each other: an unsynchronised LDS slot reuse shows up here as run-to-run differences."""
    import iree_turbine_amd as ita
    from oracle import inputs

    announce(f"attention repeatability causal={causal}")
    q, k, v = [t.to(dev) for t in inputs.attention_inputs(2, 32, 4096, 128)]
    outs = []
    for variant in range(len(ita._lib.variants("flash_attn_fwd"))):
        first = torch.empty_like(q)
        ita.launch.flash_attn_fwd_out(q, k, v, first, causal, 0.0, variant)
        for _ in range(3):
            again = torch.empty_like(q)
            ita.launch.flash_attn_fwd_out(q, k, v, again, causal, 0.0, variant)
            assert torch.equal(first, again), f"variant {variant} differs between launches"
        outs.append(first.float())
    for other in outs[1:]:
        torch.testing.assert_close(outs[0], other, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("layout", ["bshd", "packed_qkv", "head_slice"])
def test_attention_strided_operands(dev, layout, causal):
    """Transposed [B, S, H, D] views, slices of one packed QKV projection and head slices are read in place
    (no copies) and give what the contiguous tensors give."""
    import iree_turbine_amd  # noqa: F401
    from oracle import attention as oa, inputs

    B, H, S, D = 2, 4, 200, 128
    announce(f"flash_attn_fwd strided layout={layout} causal={causal}")
    q, k, v = inputs.attention_inputs(B, H, S, D, seed=21)
    if layout == "bshd":
        dq, dk, dv = (t.to(dev).transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v))
    elif layout == "packed_qkv":
        packed = torch.stack([t.transpose(1, 2) for t in (q, k, v)], dim=2).contiguous().to(dev)  # [B, S, 3, H, D]
        dq, dk, dv = (packed[:, :, i].transpose(1, 2) for i in range(3))
    else:
        wide = [torch.randn(B, H + 3, S, D, dtype=torch.float16, device=dev) for _ in range(3)]
        for w, t in zip(wide, (q, k, v)):
            w[:, 2:2 + H] = t.to(dev)
        dq, dk, dv = (w[:, 2:2 + H] for w in wide)
    assert not dq.is_contiguous()
    o = torch.ops.mi355.flash_attn_fwd(dq, dk, dv, causal, 0.0)
    torch.cuda.synchronize()
    if layout != "head_slice":
        assert o.transpose(1, 2).is_contiguous()  # laid out like q: [B, S, H, D] in memory
    ref = oa.sdpa_ref(q, k, v, is_causal=causal)
    torch.testing.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    # bit-identical to the contiguous call: the layout changes addresses only
    oc = torch.ops.mi355.flash_attn_fwd(q.to(dev), k.to(dev), v.to(dev), causal, 0.0)
    assert torch.equal(o.contiguous(), oc)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("H,Hkv", [(8, 2), (8, 1), (16, 8), (6, 3)])
def test_attention_grouped_kv_heads(dev, H, Hkv, causal):
    """Query head h reads K/V head h // (H // Hkv): equal to attention over K/V repeated per group."""
    import iree_turbine_amd  # noqa: F401
    from oracle import attention as oa, inputs

    B, S, D = 2, 160, 128
    announce(f"flash_attn_fwd gqa H={H} Hkv={Hkv} causal={causal}")
    q, _, _ = inputs.attention_inputs(B, H, S, D, seed=31)
    _, k, v = inputs.attention_inputs(B, Hkv, S, D, seed=32)
    o = torch.ops.mi355.flash_attn_fwd(q.to(dev), k.to(dev), v.to(dev), causal, 0.0)
    torch.cuda.synchronize()
    kr, vr = (t.repeat_interleave(H // Hkv, dim=1) for t in (k, v))
    torch.testing.assert_close(o.float().cpu(), oa.sdpa_ref(q, kr, vr, is_causal=causal), rtol=RTOL, atol=ATOL)
    if Hkv == 1:  # a broadcast (head stride 0) view of the single K/V head is the same computation
        o2 = torch.ops.mi355.flash_attn_fwd(q.to(dev), k.to(dev).expand(B, H, S, D), v.to(dev).expand(B, H, S, D), causal, 0.0)
    else:
        o2 = torch.ops.mi355.flash_attn_fwd(q.to(dev), kr.to(dev), vr.to(dev), causal, 0.0)
    assert torch.equal(o, o2)


def test_attention_strided_c_abi_errors(dev):
    """The strided entry point rejects what the kernel cannot address."""
    import ctypes
    from iree_turbine_amd import _lib

    lib = _lib.load()
    t = torch.zeros(1, 1, 16, 128, dtype=torch.float16, device=dev)
    arr = lambda *s: (ctypes.c_int64 * 3)(*s)
    good = arr(2048, 2048, 128)
    call = lambda qs, os_, hkv=1, h=1, b=1: lib.mi355_flash_attn_fwd_strided(
        t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), b, h, hkv, 16, 16, 128, qs, good, good, os_, 0.1, 0, -1, None)
    assert call(arr(2048, 2048, 100), good) < 0   # row stride not a multiple of 8 and < 128
    assert call(arr(2048, 2048, 64), good) < 0    # rows would overlap
    assert call(arr(2048, -8, 128), good) < 0     # negative stride
    assert call(good, arr(0, 2048, 128), b=2) < 0  # output batch stride 0 with two batches
    assert call(good, good, hkv=2, h=3) < 0       # heads not divisible
    assert b"flash_attn_fwd_strided" in lib.mi355_last_error()


def test_attention_contract_errors(dev):
    import iree_turbine_amd  # noqa: F401

    q = torch.zeros(1, 1, 16, 64, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.flash_attn_fwd(q, q, q, False, 0.0)  # D = 64
    q = torch.zeros(1, 1, 16, 128, dtype=torch.float32, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.flash_attn_fwd(q, q, q, False, 0.0)
