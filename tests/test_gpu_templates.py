"""GPU: the template getters / launchable surface and stream ordering, through the C ABI."""

import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu


def test_template_kernels_write_outputs_in_place(dev):
    import iree_turbine_amd as ita
    from iree_turbine_amd.templates import (AttentionShape, get_gemm_kernel, get_mxfp4_gemm_kernel,
                                             get_paged_decode_attention_kernels, get_vanilla_attention_kernel,
                                             paged_decode_attention_shape)
    from oracle import attention as oa, gemm as og, inputs, mxfp4 as om, paged_decode as op

    announce("templates: gemm")
    a, b = inputs.gemm_inputs(256, 384, 128)
    kern, hp = get_gemm_kernel((256, 384, 128))
    gemm = ita.wave_compile(ita.WaveCompileOptions(subs=hp), kern)
    c = torch.zeros(256, 384, dtype=torch.float32, device=dev)
    ret = gemm(a.to(dev), b.to(dev), c)
    assert ret is c
    torch.testing.assert_close(c.cpu(), og.gemm_nt_ref(a, b), rtol=1e-2, atol=1e-2)
    # non-contiguous inputs are made contiguous (runtime/launch.py:215-216)
    at = a.t().contiguous().to(dev).t()
    assert not at.is_contiguous()
    c2 = torch.zeros_like(c)
    gemm(at, b.to(dev), c2)
    assert torch.equal(c2, c)

    announce("templates: attention")
    q, k, v = inputs.attention_inputs(1, 2, 200, 128)
    shape = AttentionShape(num_query_heads=2, num_kv_heads=2, head_size=128, head_size_kv=128, query_seq_len=200, kv_seq_len=200)
    for causal in (False, True):
        kern, hp = get_vanilla_attention_kernel(shape, is_causal=causal)
        fa = ita.wave_compile(ita.WaveCompileOptions(subs=hp), kern)
        o = torch.zeros(1, 2, 200, 128, dtype=torch.float16, device=dev)
        fa(q.to(dev), k.to(dev), v.to(dev), o)
        torch.testing.assert_close(o.float().cpu(), oa.sdpa_ref(q, k, v, causal), rtol=1e-2, atol=2e-3)

    announce("templates: paged decode two phases")
    dq, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=3, min_len=20, max_len=600, seed=2)
    dshape = paged_decode_attention_shape(32, 8, 128, 128, 16, 3)
    p0, p1, hp0, hp1 = get_paged_decode_attention_kernels(dshape, num_kv_splits=4, k_shape=kc.shape, v_shape=vc.shape)
    p0 = ita.wave_compile(ita.WaveCompileOptions(subs=hp0), p0)
    p1 = ita.wave_compile(ita.WaveCompileOptions(subs=hp1), p1)
    pacc = torch.empty(3, 32, 4, 128, dtype=torch.float32, device=dev)
    pml = torch.empty(3, 32, 4, 2, dtype=torch.float32, device=dev)
    out = torch.empty(3, 32, 128, dtype=torch.float16, device=dev)
    p0(dq.to(dev), kc.to(dev), vc.to(dev), bt.to(dev), sl.to(dev), pacc, pml)
    p1(pacc, pml, out)
    torch.testing.assert_close(out.float().cpu(), op.paged_decode_ref(dq, kc, vc, bt, sl), rtol=1e-2, atol=2e-3)

    announce("templates: mxfp4")
    ma, mas, mb, mbs = inputs.mxfp4_inputs(128, 256, 512)
    kern, hp = get_mxfp4_gemm_kernel((128, 256, 512))
    mx = ita.wave_compile(ita.WaveCompileOptions(subs=hp), kern)
    mc = torch.empty(128, 256, dtype=torch.bfloat16, device=dev)
    mx(ma.to(dev), mas.to(dev), mb.to(dev), mbs.to(dev), mc)
    ref = om.mxfp4_gemm_ref(ma, mas, mb, mbs)
    assert ((mc.float().cpu() - ref).norm() / ref.norm()).item() < 1e-2


def test_launches_are_ordered_on_the_current_stream(dev):
    """Two dependent GEMMs on two side streams chained by events, repeated, then a non-blocking copy and
    one synchronize -- the pattern of tests/runtime/device_stream_test.py:42-86."""
    import iree_turbine_amd  # noqa: F401

    announce("stream ordering")
    n = 256
    ones = torch.ones(n, n, dtype=torch.float16, device=dev) / 16  # (x @ ones^T / 16) keeps magnitudes at n/16 * x
    x = torch.eye(n, dtype=torch.float16, device=dev)
    s1, s2 = torch.cuda.Stream(dev), torch.cuda.Stream(dev)
    results = []
    for _ in range(20):
        s1.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(s1):
            y = torch.ops.mi355.gemm_nt(x, ones, "float16", -1)       # row sums of I / 16 = 1/16
            ev = torch.cuda.Event()
            ev.record(s1)
        with torch.cuda.stream(s2):
            s2.wait_event(ev)
            z = torch.ops.mi355.gemm_nt(y, ones, "float16", -1)       # n * (1/16) * (1/16) = 1
            results.append(z.to("cpu", non_blocking=True))
    torch.cuda.synchronize()
    for z in results:
        assert torch.equal(z, torch.ones(n, n, dtype=torch.float16))
