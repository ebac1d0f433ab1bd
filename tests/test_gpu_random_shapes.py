"""GPU parity on seeded random shapes: every kernel family against its oracle over a few dozen draws that mix
aligned and ragged sizes, head ratios, page sizes, split counts and windows -- the combinations the hand-picked
cases of the other files do not enumerate."""

import random

import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu


def _rel(got, ref):
    ref = ref.double()
    return ((got.double().cpu() - ref).norm() / ref.norm().clamp_min(1e-30)).item()


def _dim(rng, aligned_to):
    """A size that is sometimes a tile multiple, sometimes ragged."""
    kind = rng.random()
    if kind < 0.35:
        return aligned_to * rng.randint(1, 4)
    if kind < 0.5:
        return rng.randint(1, 40)
    return rng.randint(1, 700)


def test_random_gemm(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import gemm as og, inputs

    rng = random.Random(101)
    for case in range(40):
        M, N = _dim(rng, 256), _dim(rng, 256)
        K = rng.choice([8, 16, 64, 72, 128, 192, 256, 320, 512, 1024, 1536])
        out_dtype = rng.choice(["float16", "float32"])
        announce(f"random gemm {case}: {M}x{N}x{K} {out_dtype}")
        a, b = inputs.gemm_inputs(M, N, K, seed=case)
        c = torch.ops.mi355.gemm_nt(a.to(dev), b.to(dev), out_dtype, -1)
        torch.testing.assert_close(c.float().cpu(), og.gemm_nt_ref(a, b), rtol=1e-2, atol=1e-2)


def test_random_gemm_few_tiles_long_k(dev):
    """Tile-aligned products with few 256x256 tiles and long K: the shapes the op hands a K-split workspace to (and
    their neighbours that take none), fp16 and bf16 operands, against an fp32 product of sampled rows and columns."""
    import iree_turbine_amd  # noqa: F401
    from iree_turbine_amd import _lib
    from oracle import inputs

    lib = _lib.load()
    rng = random.Random(111)
    split = 0
    for case in range(30):
        tm, tn = rng.randint(1, 12), rng.randint(1, 12)
        if case % 6 == 5:
            tm, tn = rng.choice([(8, 40), (40, 8), (16, 18), (9, 32)])  # a full round of tiles and a sparse one behind it
        M, N = 256 * tm, 256 * tn
        if case % 3 == 1:
            M, N = 128 * rng.randint(1, 9), 128 * rng.randint(1, 9)  # small products, odd multiples of 128 among them
        K = rng.choice([4096, 4224, 6144, 8192, 12288])
        dtype = rng.choice([torch.float16, torch.bfloat16])
        out_dtype = rng.choice(["float32", str(dtype).split(".")[1]])
        need = lib.mi355_gemm_nt_workspace_bytes(M, N, K)
        split += need > 0
        announce(f"random few-tile gemm {case}: {M}x{N}x{K} {dtype} -> {out_dtype}, workspace {need >> 20} MiB")
        a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K, seed=200 + case, dtype=dtype)]
        c = torch.ops.mi355.gemm_nt(a, b, out_dtype, -1)
        tol = dict(rtol=1e-3, atol=1e-3) if out_dtype == "float32" else dict(rtol=1e-2, atol=1e-2)
        rows = torch.tensor(sorted({0, M - 1, rng.randrange(M), rng.randrange(M)}), device=dev)
        cols = torch.tensor(sorted({0, N - 1, rng.randrange(N), rng.randrange(N)}), device=dev)
        torch.testing.assert_close(c[rows].float(), a[rows].float() @ b.float().t(), **tol)
        torch.testing.assert_close(c[:, cols].float(), a.float() @ b[cols].float().t(), **tol)
    assert split >= 8  # the draw does exercise the split


def test_random_gemm_small_and_mid_products(dev):
    """Products whose tile shape and K ranges the automatic choice picks by rule: multiples of 64 up to 128 tiles of
    128x128 (64x64, 128x64 or 128x128 tiles, one to eight K ranges), and 129 to 256 tiles of 256x128 -- fp16 and bf16
    operands, both output types, whole matrix against an fp32 product."""
    import iree_turbine_amd  # noqa: F401
    from iree_turbine_amd import _lib
    from oracle import inputs

    lib = _lib.load()
    rng = random.Random(333)
    split = 0
    for case in range(48):
        if case % 4 == 3:  # 129 to 256 tiles of 256x128
            tm = rng.randint(2, 12)
            tn = rng.randint(-(-129 // tm), 256 // tm)
            M, N = 256 * tm, 128 * tn
            K = 64 * rng.randint(4, 40)
        else:
            M = 64 * rng.randint(1, 32)
            N = 64 * rng.randint(1, min(32, (1 << 21) // (64 * M)))
            K = rng.choice([64, 128, 192, 320, 1024, 1088, 2048, 3072, 4096, 5120, 8192, 12288])
        dtype = rng.choice([torch.float16, torch.bfloat16])
        out_dtype = rng.choice(["float32", str(dtype).split(".")[1]])
        need = lib.mi355_gemm_nt_workspace_bytes(M, N, K)
        split += need > 0
        announce(f"random small/mid gemm {case}: {M}x{N}x{K} {dtype} -> {out_dtype}, workspace {need >> 10} KiB")
        a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K, seed=400 + case, dtype=dtype)]
        c = torch.ops.mi355.gemm_nt(a, b, out_dtype, -1)
        tol = dict(rtol=1e-3, atol=1e-3) if out_dtype == "float32" else dict(rtol=1e-2, atol=1e-2)
        torch.testing.assert_close(c.float(), a.float() @ b.float().t(), **tol)
    assert split >= 6  # the draw does exercise the split


def test_random_gemm_cut_tiles(dev):
    """Any number of rows against any multiple of 8 columns, within one round of tiles: the last tile row and column are
    cut inside the kernels, with one to eight K ranges -- fp16 and bf16 operands, both output types, whole matrix against
    an fp32 product; the launcher pads nothing."""
    import iree_turbine_amd as ita
    from iree_turbine_amd import _lib
    from oracle import inputs

    lib = _lib.load()
    rng = random.Random(4242)
    split = 0
    for case in range(40):
        if case % 4 == 3:  # beyond the small-product rule: one round of 128x128 or 256x128 tiles
            M = rng.randint(1100, 3000)
            N = 8 * rng.randint((1 << 21) // (-(-M // 64) * 64) // 8 + 1, 16 * (256 // -(-M // 256)))
            K = 64 * rng.randint(4, 24)
        elif case % 4 == 0:  # few tiles and a long K: K ranges with cut tiles
            M, N, K = rng.randint(1, 300), 8 * rng.randint(1, 80), rng.choice([2048, 4096, 8192])
        else:
            M = rng.randint(1, 1400)
            N = 8 * rng.randint(1, max(1, min(256, (1 << 21) // (-(-M // 64) * 64) // 8 - 8)))
            K = rng.choice([64, 192, 1024, 1088, 2048, 4096, 8192])
        dtype = rng.choice([torch.float16, torch.bfloat16])
        out_dtype = rng.choice(["float32", str(dtype).split(".")[1]])
        need = lib.mi355_gemm_nt_workspace_bytes(M, N, K)
        split += need > 0
        announce(f"random cut-tile gemm {case}: {M}x{N}x{K} {dtype} -> {out_dtype}, workspace {need >> 10} KiB")
        assert ita.launch._ragged_rows_fit(M, N, K), (M, N, K)
        a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K, seed=900 + case, dtype=dtype)]
        c = torch.ops.mi355.gemm_nt(a, b, out_dtype, -1)
        tol = dict(rtol=1e-3, atol=1e-3) if out_dtype == "float32" else dict(rtol=1e-2, atol=1e-2)
        torch.testing.assert_close(c.float(), a.float() @ b.float().t(), **tol)
    assert split >= 8  # the draw does exercise the split


def test_random_attention(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import attention as oa

    rng = random.Random(202)
    for case in range(30):
        B, Hkv = rng.randint(1, 3), rng.choice([1, 2, 3, 4])
        group = rng.choice([1, 1, 2, 4])
        Sq = rng.choice([1, 7, 64, 127, 128, 129, 300, 512, 777])
        causal = rng.random() < 0.5
        Sk = Sq if rng.random() < 0.6 else rng.choice([1, 33, 64, 200, 512, 1000])
        if causal and Sk < Sq:
            Sk = Sq  # fewer keys than queries leaves early queries with nothing to attend
        announce(f"random attention {case}: B{B} Hq{Hkv * group} Hkv{Hkv} Sq{Sq} Sk{Sk} causal={causal}")
        g = torch.Generator().manual_seed(case)
        q = torch.randn(B, Hkv * group, Sq, 128, generator=g).half()
        k = torch.randn(B, Hkv, Sk, 128, generator=g).half()
        v = torch.randn(B, Hkv, Sk, 128, generator=g).half()
        out = torch.ops.mi355.flash_attn_fwd(q.to(dev), k.to(dev), v.to(dev), causal, 0.0)
        kr, vr = k.repeat_interleave(group, dim=1), v.repeat_interleave(group, dim=1)
        if causal and Sk != Sq:
            # query i of the last Sq positions sees keys <= Sk - Sq + i
            s = torch.matmul(q.float(), kr.float().transpose(-1, -2)) / 128 ** 0.5
            vis = torch.arange(Sk)[None, :] <= (Sk - Sq + torch.arange(Sq))[:, None]
            ref = torch.matmul(torch.softmax(s.masked_fill(~vis, float("-inf")), dim=-1), vr.float())
        else:
            ref = oa.sdpa_ref(q, kr, vr, is_causal=causal)
        torch.testing.assert_close(out.float().cpu(), ref, rtol=1e-2, atol=2e-3)


def test_random_paged(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    rng = random.Random(303)
    for case in range(30):
        page = rng.choice([16, 16, 32, 64, 128, 256])
        Hkv = rng.choice([1, 2, 4, 8])
        group = rng.choice([1, 2, 4, 8, 16])
        S = rng.randint(1, 9)
        max_len = rng.choice([1, 15, 16, 17, 100, 600, 2000])
        splits = rng.choice([0, 1, 2, 3, 5, 8])
        window = rng.choice([0, 0, 1, 20, 64, 500])
        announce(f"random paged {case}: S{S} Hq{Hkv * group} Hkv{Hkv} page{page} max_len{max_len} splits{splits} window{window}")
        q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=S, num_q_heads=Hkv * group, num_kv_heads=Hkv, page=page,
                                                       min_len=0 if case % 3 == 0 else 1, max_len=max_len, seed=case)
        args = [t.to(dev) for t in (q, kc, vc, bt, sl)]
        if window:
            out = torch.ops.mi355.paged_decode_attn_window(*args, 0.0, splits, window)
        else:
            out = torch.ops.mi355.paged_decode_attn(*args, 0.0, splits)
        ref = op.paged_decode_ref(q, kc, vc, bt, sl, window=window)
        torch.testing.assert_close(out.float().cpu(), ref, rtol=1e-2, atol=2e-3)
        n_new = rng.choice([1, 3, 16, 50])
        qn = torch.randn(S, n_new, Hkv * group, 128, generator=torch.Generator().manual_seed(case)).half()
        pre = torch.ops.mi355.paged_prefill_attn(qn.to(dev), *args[1:], 0.0)
        torch.testing.assert_close(pre.float().cpu(), op.paged_prefill_ref(qn, kc, vc, bt, sl), rtol=1e-2, atol=2e-3)


def test_random_block_scaled_gemms(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, mxfp4 as o4, mxfp6 as o6, mxfp8 as o8

    rng = random.Random(404)
    for case in range(36):
        M, N = _dim(rng, 256), _dim(rng, 256)
        K = 32 * rng.choice([1, 2, 3, 5, 8, 16, 24, 32, 40, 64])
        out_dtype = rng.choice(["bfloat16", "float32"])
        tol = 1e-2 if out_dtype == "bfloat16" else 5e-4
        kind = case % 4
        announce(f"random mx gemm {case}: kind {kind} {M}x{N}x{K} {out_dtype}")
        if kind == 0:
            a, asc, b, bsc = inputs.mxfp4_inputs(M, N, K, seed=case)
            got, ref = torch.ops.mi355.mxfp4_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), out_dtype, -1), o4.mxfp4_gemm_ref(a, asc, b, bsc)
        elif kind == 1:
            a, asc, b, bsc = inputs.mxfp8_inputs(M, N, K, seed=case)
            got, ref = torch.ops.mi355.mxfp8_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), out_dtype, -1), o8.mxfp8_gemm_ref(a, asc, b, bsc)
        elif kind == 2:
            fmt = rng.choice(["e2m3", "e3m2"])
            a, asc, b, bsc = inputs.mxfp6_inputs(M, N, K, seed=case)
            got = torch.ops.mi355.mxfp6_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), fmt, out_dtype, -1)
            ref = o6.mxfp6_gemm_ref(a, asc, b, bsc, fmt)
        else:
            a, _, b, _ = inputs.mxfp8_inputs(M, N, K, seed=case)
            got, ref = torch.ops.mi355.fp8_gemm(a.to(dev), b.to(dev), 0.5, out_dtype, -1), o8.fp8_gemm_ref(a, b, 0.5)
        assert _rel(got, ref) < tol, (case, kind, M, N, K)


def test_random_quantisers(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp4 as o4, mxfp6 as o6, mxfp8 as o8

    rng = random.Random(505)
    for case in range(30):
        rows, K = rng.randint(1, 300), 32 * rng.randint(1, 70)
        dtype = rng.choice([torch.float16, torch.bfloat16, torch.float32])
        announce(f"random quantise {case}: {rows}x{K} {dtype}")
        g = torch.Generator().manual_seed(case)
        x = (torch.randn(rows, K, generator=g) * torch.exp(torch.randn(rows, 1, generator=g) * 4)).to(dtype)
        if dtype != torch.float32:
            x = torch.nan_to_num(x, posinf=6e4, neginf=-6e4)
        c, s = torch.ops.mi355.mxfp4_quantize(x.to(dev))
        rc, rs = o4.mxfp4_quantize_ref(x)
        assert np.array_equal(c.cpu().numpy(), rc) and np.array_equal(s.cpu().numpy(), rs)
        c, s = torch.ops.mi355.mxfp8_quantize(x.to(dev))
        rc, rs = o8.mxfp8_quantize_ref(x)
        assert np.array_equal(c.cpu().numpy(), rc) and np.array_equal(s.cpu().numpy(), rs)
        fmt = rng.choice(["e2m3", "e3m2"])
        c, s = torch.ops.mi355.mxfp6_quantize(x.to(dev), fmt)
        rc, rs = o6.mxfp6_quantize_ref(x, fmt)
        assert np.array_equal(c.cpu().numpy(), rc) and np.array_equal(s.cpu().numpy(), rs)
