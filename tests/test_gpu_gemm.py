"""GPU parity: fp16 NT GEMM through the C ABI vs the CPU oracle (torch fp32 matmul), rtol = atol = 1e-2."""

import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

RTOL = ATOL = 1e-2  # the contract tolerance for the fp16 GEMM


def _run(dev, M, N, K, out_dtype, variant=-1, seed=10):
    import iree_turbine_amd as ita
    from oracle import gemm as og, inputs

    announce(f"gemm_nt M={M} N={N} K={K} out={out_dtype} variant={variant} seed={seed}")
    a, b = inputs.gemm_inputs(M, N, K, seed=seed)
    c = torch.ops.mi355.gemm_nt(a.to(dev), b.to(dev), out_dtype, variant)
    torch.cuda.synchronize()
    ref = og.gemm_nt_ref(a, b)
    return c.float().cpu(), ref


@pytest.mark.parametrize("variant", [-1, 0, 1, 2, 4, 5, 6, 7, 8, 9])  # every tiled kernel (3 is the skinny-M kernel, 10 the any-shape one)
def test_gemm_1024_f32_all_variants(dev, variant):
    c, ref = _run(dev, 1024, 1024, 1024, "float32", variant)
    torch.testing.assert_close(c, ref, rtol=RTOL, atol=ATOL)
    # fp32 output of an fp32-accumulating kernel should be much closer than the stated tolerance
    assert (c - ref).abs().max().item() < 1e-3


@pytest.mark.parametrize("shape", [(256, 256, 64), (512, 768, 192), (2048, 1024, 4096), (128, 384, 640)])
@pytest.mark.parametrize("out_dtype", ["float32", "float16"])
def test_gemm_tiled_shapes(dev, shape, out_dtype):
    c, ref = _run(dev, *shape, out_dtype)
    torch.testing.assert_close(c, ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("shape", [(16, 16, 16), (32, 32, 32), (1, 1, 1), (65, 33, 17), (100, 200, 72), (3, 129, 257), (64, 64, 8)])
def test_gemm_ragged_shapes(dev, shape):
    # the reference's own smoke sizes are 16^3 / 32^3 (tests/kernel/boo/driver/numerics_smoke_test.py:473-520)
    c, ref = _run(dev, *shape, "float32")
    torch.testing.assert_close(c, ref, rtol=RTOL, atol=ATOL)
    c16, _ = _run(dev, *shape, "float16")
    torch.testing.assert_close(c16, ref, rtol=RTOL, atol=ATOL)


def test_gemm_identity_and_ones(dev):
    import iree_turbine_amd  # noqa: F401

    announce("gemm identity / block of ones")
    M = K = 512
    N = 256
    b = (torch.randn(N, K) * 0.5).half()
    eye = torch.eye(M, K).half()
    c = torch.ops.mi355.gemm_nt(eye.to(dev), b.to(dev), "float16", -1).cpu()
    assert torch.equal(c, b.t().contiguous())  # A = I  =>  C = B^T exactly
    # structured block-of-ones (the idea of numerics.py:319-338): integer sums are exact
    a1 = torch.zeros(256, 1024).half()
    a1[32:96, 100:612] = 1
    b1 = torch.zeros(256, 1024).half()
    b1[:, 300:900] = 1
    c1 = torch.ops.mi355.gemm_nt(a1.to(dev), b1.to(dev), "float32", -1).cpu()
    exp = torch.zeros(256, 256)
    exp[32:96, :] = 612 - 300
    assert torch.equal(c1, exp)


def test_gemm_error_statistics(dev):
    """The reference's three-way criteria (numerics.py:266-316): no drift, and an error spread no worse
    than 1.2x torch's own GPU GEMM, both measured against an fp64 CPU result."""
    from oracle import gemm as og, inputs, numerics as on

    announce("gemm error statistics 1024x1024x2048")
    a, b = inputs.gemm_inputs(1024, 1024, 2048, seed=3)
    ref64 = og.gemm_nt_f64(a, b)
    ours = torch.ops.mi355.gemm_nt(a.to(dev), b.to(dev), "float16", -1).cpu()
    theirs = torch.mm(a.to(dev), b.to(dev).t()).cpu()
    e_ours, nan1 = on.element_errors(ours, ref64)
    e_theirs, nan2 = on.element_errors(theirs, ref64)
    s_ours, s_theirs = on.error_statistics(e_ours), on.error_statistics(e_theirs)
    assert not nan1 and not nan2
    assert on.mean_near_zero(s_ours), s_ours
    assert on.stddev_ratio_ok(s_ours, s_theirs), (s_ours, s_theirs)


def test_gemm_contract_errors(dev):
    import iree_turbine_amd  # noqa: F401

    a = torch.zeros(64, 64, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a, torch.zeros(64, 32, dtype=torch.float16, device=dev), "float32", -1)
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a.float(), a.float(), "float32", -1)
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a, a, "float32", 0)  # 256x256 tile does not divide 64x64
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a, a, "float32", 99)  # no such variant
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a, a, "int8", -1)


@pytest.mark.parametrize("shape", [(8192, 8192, 8192), (4096, 4096, 4096), (2048, 10240, 8192), (2048, 57344, 8192)])
def test_gemm_full_size_properties(dev, shape):
    """At benchmark sizes: sampled rows/columns against the fp32 oracle, plus linearity in A."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs

    M, N, K = shape
    announce(f"gemm full size {shape}")
    a, b = inputs.gemm_inputs(M, N, K)
    ad, bd = a.to(dev), b.to(dev)
    c = torch.ops.mi355.gemm_nt(ad, bd, "float16", -1)
    rows = torch.tensor([0, 1, 255, 256, M // 2 + 7, M - 1])
    cols = torch.tensor([0, 31, 32, 257, N // 2 + 3, N - 1])
    ref_rows = a[rows].float() @ b.float().t()
    torch.testing.assert_close(c[rows.to(dev)].float().cpu(), ref_rows, rtol=RTOL, atol=ATOL)
    ref_cols = a.float() @ b[cols].float().t()
    torch.testing.assert_close(c[:, cols.to(dev)].float().cpu(), ref_cols, rtol=RTOL, atol=ATOL)
    # linearity: (2A) B^T == 2 (A B^T) bit for bit with fp32 output (doubling is exact in every
    # product and partial sum; fp16 output would differ where results round into subnormals)
    c32 = torch.ops.mi355.gemm_nt(ad, bd, "float32", -1)
    c2 = torch.ops.mi355.gemm_nt(ad * 2, bd, "float32", -1)
    assert torch.equal(c2, c32 * 2)
    assert torch.equal(c32.half(), c)  # the fp16 epilogue is round-to-nearest-even of the fp32 result


@pytest.mark.parametrize("shape", [(8192, 8192, 8192), (2048, 10240, 8192), (2048, 57344, 8192)])
def test_gemm_full_size_repeatable(dev, shape):
    """Whole-matrix checks at benchmark sizes: every tiled variant is bit-identical across launches (an
    unsynchronised LDS stage reuse would differ from run to run) and agrees with the simple generic kernel."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"gemm repeatability {shape}")
    a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K)]
    names = ita._lib.variants("gemm_f16_nt")
    generic = torch.ops.mi355.gemm_nt(a, b, "float32", len(names) - 1)
    by_name = {}
    for variant in range(len(names) - 1):
        if names[variant].startswith("skinny"):
            continue  # M <= 32 only: covered by test_gemm_skinny_m
        first = torch.ops.mi355.gemm_nt(a, b, "float32", variant)
        for _ in range(2):
            assert torch.equal(first, torch.ops.mi355.gemm_nt(a, b, "float32", variant)), names[variant]
        torch.testing.assert_close(first, generic, rtol=1e-3, atol=1e-3)
        if names[variant].startswith(("staged", "stream")):
            by_name[names[variant]] = first
        del first
    # the tail split hands the last tile columns to a second kernel that adds K in the same order: the whole matrix
    # equals the unsplit streamed kernel's bit for bit, and so does the same kernel launched with one workgroup per
    # CU, walking its tiles as one slab sequence
    streamed = [v for k, v in sorted(by_name.items()) if k.startswith("stream")]
    assert len(streamed) == 3 and torch.equal(streamed[0], streamed[1]) and torch.equal(streamed[0], streamed[2])
    # and the register-staged kernel, an independent implementation (other MFMA shape, other load path) that adds K
    # in the same order per element
    staged = [v for k, v in sorted(by_name.items()) if k.startswith("staged")]
    assert len(staged) == 1 and torch.equal(staged[0], streamed[0])


@pytest.mark.parametrize("shape", [(4096, 4608, 192), (4352, 4352, 128), (8192, 8704, 320), (512, 256, 4096)])
@pytest.mark.parametrize("out_dtype", ["float16", "float32"])
def test_gemm_persistent_tile_walk(dev, shape, out_dtype):
    """The persistent kernel walks several tiles per workgroup as one slab sequence: more tiles than CUs,
    tile counts that are not multiples of 8 or of the grid, odd slab counts (the LDS stage parity flips
    between tiles), the minimum of two slabs, and fewer tiles than CUs -- whole matrix against the
    independent generic kernel."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"gemm persistent walk {shape} {out_dtype}")
    names = ita._lib.variants("gemm_f16_nt")
    assert names[0].startswith("persistent")
    a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K)]
    got = torch.ops.mi355.gemm_nt(a, b, out_dtype, 0)
    ref = torch.ops.mi355.gemm_nt(a, b, out_dtype, len(names) - 1)
    torch.testing.assert_close(got.float(), ref.float(), rtol=1e-3, atol=1e-3)
    rows = torch.tensor([0, 255, 256, M - 1])
    exact = a[rows.to(dev)].float() @ b.float().t()
    torch.testing.assert_close(got[rows.to(dev)].float(), exact, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("out_dtype", ["float16", "float32"])
@pytest.mark.parametrize("shape", [(256, 256, 256), (512, 768, 384), (1024, 512, 1152), (2048, 10240, 512)])
def test_gemm_staged_slab_rotation(dev, shape, out_dtype):
    """The register-staged kernel keeps three slabs in flight in two alternating register sets: the minimum of
    four slabs, slab counts that are 2 and 0 mod 4 (the loop is written for pairs), a ragged tile grid and a
    grid larger than the chip -- whole matrix against the independent generic kernel, rows against fp32."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"gemm staged {shape} {out_dtype}")
    names = ita._lib.variants("gemm_f16_nt")
    v = next(i for i, n in enumerate(names) if n.startswith("staged"))
    a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K)]
    got = torch.ops.mi355.gemm_nt(a, b, out_dtype, v)
    ref = torch.ops.mi355.gemm_nt(a, b, out_dtype, len(names) - 1)
    torch.testing.assert_close(got.float(), ref.float(), rtol=1e-3, atol=1e-3)
    rows = torch.tensor([0, 127, 128, M - 1])
    exact = a[rows.to(dev)].float() @ b.float().t()
    torch.testing.assert_close(got[rows.to(dev)].float(), exact, rtol=RTOL, atol=ATOL)
    assert torch.equal(got, torch.ops.mi355.gemm_nt(a, b, out_dtype, v))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("out32", [False, True])
@pytest.mark.parametrize("shape", [(128, 128, 4096), (256, 384, 4160), (1024, 1024, 4096), (2048, 1536, 2048), (2048, 1536, 2112),
                                   (2048, 2048, 8192), (2048, 2176, 4096), (128, 256, 1984)])
def test_gemm_pipelined_ring_depth(dev, shape, out32, dtype):
    """The 128x128 kernel takes its slab form (whole-slab fragment sets, four slabs in LDS) when every workgroup has a CU
    to itself and its k-step form (two slabs) beyond 256 tiles: one tile, even and odd slab counts (64, 65, 33, 31: the
    slab loop is unrolled by two), tile counts on both sides of the limit (192 and 256 against 272) -- whole matrix
    against the independent generic kernel, rows against fp32, launches repeat bit for bit."""
    import iree_turbine_amd as ita

    M, N, K = shape
    announce(f"gemm pipelined ring {shape} {dtype} out32={out32}")
    names = ita._lib.variants("gemm_f16_nt")
    v = next(i for i, n in enumerate(names) if n.startswith("pipelined"))
    g = torch.Generator().manual_seed(M + 3 * N + 7 * K)
    a = (torch.randn(M, K, generator=g) * 0.25).to(dtype).to(dev)
    b = (torch.randn(N, K, generator=g) * 0.25).to(dtype).to(dev)
    out_dtype = "float32" if out32 else str(dtype).replace("torch.", "")
    got = torch.ops.mi355.gemm_nt(a, b, out_dtype, v)
    ref = torch.ops.mi355.gemm_nt(a, b, out_dtype, len(names) - 1)
    tol = 1e-3 if (out32 or dtype == torch.float16) else 8e-3
    torch.testing.assert_close(got.float(), ref.float(), rtol=tol, atol=tol * 4)
    rows = torch.tensor([0, 63, 64, M - 1])
    exact = a[rows.to(dev)].float() @ b.float().t()
    torch.testing.assert_close(got[rows.to(dev)].float(), exact, rtol=RTOL, atol=ATOL)
    assert torch.equal(got, torch.ops.mi355.gemm_nt(a, b, out_dtype, v))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("out32", [False, True])
@pytest.mark.parametrize("shape", [(256, 128, 64), (512, 256, 128), (256, 384, 192), (768, 640, 320), (2048, 2560, 2048), (2048, 4096, 1600),
                                   (1024, 8192, 4096), (2304, 1792, 1536)])
def test_gemm_pipelined_256x128(dev, shape, out32, dtype):
    """The 256x128 tile of the pipelined kernel (slab form, three slabs in LDS): one tile and one slab, two, three and
    five slabs (shorter than, equal to and just beyond the ring), an odd slab count (25), and the shapes the automatic
    choice gives it (129 to 256 tiles, 256 <= K < 8192; 126 tiles: not) -- by index and through the automatic choice,
    whole matrix against the independent generic kernel, rows against fp32, launches repeat bit for bit."""
    import iree_turbine_amd as ita

    M, N, K = shape
    announce(f"gemm pipelined 256x128 {shape} {dtype} out32={out32}")
    names = ita._lib.variants("gemm_f16_nt")
    g = torch.Generator().manual_seed(M + 5 * N + 11 * K)
    a = (torch.randn(M, K, generator=g) * 0.25).to(dtype).to(dev)
    b = (torch.randn(N, K, generator=g) * 0.25).to(dtype).to(dev)
    out_dtype = "float32" if out32 else str(dtype).replace("torch.", "")
    ref = torch.ops.mi355.gemm_nt(a, b, out_dtype, len(names) - 1)
    rows = torch.tensor([0, 127, 128, M - 1], device=dev)
    exact = a[rows].float() @ b.float().t()
    tol = 1e-3 if (out32 or dtype == torch.float16) else 8e-3
    for v in (names.index("pipelined_256x128x64_w2x2"), -1):
        got = torch.ops.mi355.gemm_nt(a, b, out_dtype, v)
        torch.testing.assert_close(got.float(), ref.float(), rtol=tol, atol=tol * 4)
        torch.testing.assert_close(got[rows].float(), exact, rtol=RTOL, atol=ATOL)
        assert torch.equal(got, torch.ops.mi355.gemm_nt(a, b, out_dtype, v))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("out32", [False, True])
@pytest.mark.parametrize("shape", [(64, 64, 64), (128, 64, 128), (192, 320, 1024), (1024, 1024, 1024), (512, 512, 4096), (1024, 2048, 2048),
                                   (320, 448, 2560), (1024, 1024, 4096), (1024, 2048, 512), (64, 1024, 192), (1408, 1408, 1024)])
def test_gemm_small_products(dev, shape, out32, dtype):
    """Products of at most 128 tiles of 128x128 take 64x64, 128x64 or 128x128 tiles and one to eight K ranges by a cost
    model: one tile and one slab, two and three slabs (shorter than the ring), shapes that are no multiple of 128, each
    tile shape with and without a split, the largest size of the rule and the first beyond it (1408^2) -- the automatic
    choice through the op (which brings the workspace) and the two small-tile kernels by index, whole matrix against the
    independent generic kernel, rows against fp32, launches repeat bit for bit."""
    import iree_turbine_amd as ita

    M, N, K = shape
    announce(f"gemm small product {shape} {dtype} out32={out32}")
    names = ita._lib.variants("gemm_f16_nt")
    g = torch.Generator().manual_seed(5 * M + 3 * N + K)
    a = (torch.randn(M, K, generator=g) * 0.25).to(dtype).to(dev)
    b = (torch.randn(N, K, generator=g) * 0.25).to(dtype).to(dev)
    out_dtype = "float32" if out32 else str(dtype).replace("torch.", "")
    ref = torch.ops.mi355.gemm_nt(a, b, out_dtype, len(names) - 1)
    rows = torch.tensor([0, 63, M - 64, M - 1], device=dev)
    exact = a[rows].float() @ b.float().t()
    tol = 1e-3 if (out32 or dtype == torch.float16) else 8e-3
    for v in [-1, names.index("pipelined_64x64x64_w2x2")] + ([names.index("pipelined_128x64x64_w2x2")] if M % 128 == 0 else []):
        got = torch.ops.mi355.gemm_nt(a, b, out_dtype, v)
        torch.testing.assert_close(got.float(), ref.float(), rtol=tol, atol=tol * 4)
        torch.testing.assert_close(got[rows].float(), exact, rtol=RTOL, atol=ATOL)
        assert torch.equal(got, torch.ops.mi355.gemm_nt(a, b, out_dtype, v))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("out32", [False, True])
@pytest.mark.parametrize("shape", [(1, 64, 64), (65, 64, 128), (127, 128, 192), (129, 1024, 1024), (200, 4096, 1024), (300, 2048, 2048),
                                   (130, 8192, 1024), (1000, 2048, 512), (63, 1984, 4096), (1023, 1024, 64),
                                   (1500, 2048, 1024), (2000, 2048, 2048), (1100, 4096, 1024), (1793, 4096, 512), (1152, 4096, 1088),
                                   (200, 512, 8192), (65, 64, 4096), (700, 640, 2048)])
def test_gemm_ragged_rows(dev, shape, out32, dtype):
    """Any number of rows in the small-product range (N and K multiples of 64) and beyond it where one round of 128x128 or
    256x128 tiles covers the product: the last tile row is cut inside the kernel -- its loads of A take row
    min(row, M - 1), its stores stop at M -- on 64x64, 128x64, 128x128 and 256x128 tiles: one row, one row more and one
    row fewer than a tile, one slab and many, 1152 rows on 256x128 tiles, and few tiles with a long K, which split K (the
    partial products are whole tiles in the workspace, the merge takes the rows below M).  Whole matrix against an fp32 product, the
    rows behind the result untouched, launches repeat bit for bit."""
    import iree_turbine_amd as ita
    from iree_turbine_amd import _lib

    M, N, K = shape
    announce(f"gemm ragged rows {shape} {dtype} out32={out32}")
    g = torch.Generator().manual_seed(M + 2 * N + 3 * K)
    a = (torch.randn(M, K, generator=g) * 0.25).to(dtype).to(dev)
    b = (torch.randn(N, K, generator=g) * 0.25).to(dtype).to(dev)
    odt = torch.float32 if out32 else dtype
    full = torch.full((M + 130, N), float("nan"), dtype=odt, device=dev)
    c = full[:M]
    ita.launch.gemm_nt_out(a, b, c, -1)
    tol = dict(rtol=1e-3, atol=1e-3) if out32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(c.float(), a.float() @ b.float().t(), **tol)
    assert torch.isnan(full[M:]).all()  # nothing stored behind row M - 1
    again = torch.empty_like(c)
    ita.launch.gemm_nt_out(a, b, again, -1)
    assert torch.equal(c, again)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("out32", [False, True])
@pytest.mark.parametrize("shape", [(64, 8, 64), (64, 72, 128), (128, 136, 128), (100, 1000, 512), (512, 1000, 1024), (1024, 1016, 1024),
                                   (256, 264, 2048), (1000, 1096, 4096), (200, 4104, 1024), (2048, 2056, 1024), (1793, 3976, 512),
                                   (128, 24584, 256), (256, 1000, 4096), (100, 200, 8192), (520, 520, 2048)])
def test_gemm_ragged_columns(dev, shape, out32, dtype):
    """Any multiple of 8 columns where one round of tiles covers the product: the last tile column is cut inside the kernel
    -- its loads of B take row min(row, N - 1), its stores stop at column N -- alone and together with a cut tile row, on
    64x64, 128x64, 128x128 and 256x128 tiles: fewer columns than a tile, one 16-byte chunk more and fewer than a tile, one
    slab and many.  Whole matrix against an fp32 product (a store right of column N would land in the next row), the
    rows behind the result untouched, launches repeat bit for bit; the launcher pads nothing."""
    import iree_turbine_amd as ita
    from iree_turbine_amd import _lib

    M, N, K = shape
    announce(f"gemm ragged columns {shape} {dtype} out32={out32}")
    assert ita.launch._ragged_rows_fit(M, N, K)
    g = torch.Generator().manual_seed(M + 2 * N + 3 * K)
    a = (torch.randn(M, K, generator=g) * 0.25).to(dtype).to(dev)
    b = (torch.randn(N, K, generator=g) * 0.25).to(dtype).to(dev)
    odt = torch.float32 if out32 else dtype
    full = torch.full((M + 130, N), float("nan"), dtype=odt, device=dev)
    c = full[:M]
    ita.launch.gemm_nt_out(a, b, c, -1)
    tol = dict(rtol=1e-3, atol=1e-3) if out32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(c.float(), a.float() @ b.float().t(), **tol)
    assert torch.isnan(full[M:]).all()  # nothing stored behind row M - 1
    again = torch.empty_like(c)
    ita.launch.gemm_nt_out(a, b, again, -1)
    assert torch.equal(c, again)


@pytest.mark.parametrize("shape", [(1088, 2112, 2048), (1152, 2112, 1024), (2112, 1152, 1024)])
def test_gemm_multiples_of_64_beyond_the_small_rule(dev, shape):
    """Products too large for the small-product rule that divide by 64 and not by 128 (and too small for the launcher to
    pad them) take the 64x64 or the 128x64 tile rather than the bounds-checked kernel: whole matrix against that kernel
    and against an fp32 product."""
    import iree_turbine_amd as ita

    M, N, K = shape
    announce(f"gemm multiples of 64 {shape}")
    names = ita._lib.variants("gemm_f16_nt")
    g = torch.Generator().manual_seed(M + N + K)
    a = (torch.randn(M, K, generator=g) * 0.25).half().to(dev)
    b = (torch.randn(N, K, generator=g) * 0.25).half().to(dev)
    got = torch.ops.mi355.gemm_nt(a, b, "float32", -1)
    tile = "pipelined_128x64x64_w2x2" if M % 128 == 0 else "pipelined_64x64x64_w2x2"
    assert torch.equal(got, torch.ops.mi355.gemm_nt(a, b, "float32", names.index(tile)))  # the automatic choice is that kernel
    torch.testing.assert_close(got, torch.ops.mi355.gemm_nt(a, b, "float32", len(names) - 1), rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(got, a.float() @ b.float().t(), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("out_dtype", ["float16", "float32"])
@pytest.mark.parametrize("shape", [(256, 256, 256), (512, 768, 384), (1024, 512, 1152), (2048, 10240, 512), (4352, 4352, 640)])
def test_gemm_stream_slab_rotation(dev, shape, out_dtype):
    """The streamed kernel keeps B in three rotating LDS buffers and A in two, with loads two slabs ahead of the reads:
    the minimum of four slabs, slab counts that are 2 and 0 mod 4 and 0, 1 and 2 mod 3 (4, 6, 18, 8, 10: the loop is
    written for pairs, the B buffers rotate in threes), a ragged tile grid and grids larger than the chip -- whole
    matrix against the independent generic kernel, rows against fp32, launches repeat bit for bit."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"gemm streamed {shape} {out_dtype}")
    names = ita._lib.variants("gemm_f16_nt")
    v = names.index("stream_256x256x64_w2x2")
    a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K)]
    got = torch.ops.mi355.gemm_nt(a, b, out_dtype, v)
    ref = torch.ops.mi355.gemm_nt(a, b, out_dtype, len(names) - 1)
    torch.testing.assert_close(got.float(), ref.float(), rtol=1e-3, atol=1e-3)
    rows = torch.tensor([0, 127, 128, M - 1])
    exact = a[rows.to(dev)].float() @ b.float().t()
    torch.testing.assert_close(got[rows.to(dev)].float(), exact, rtol=RTOL, atol=ATOL)
    assert torch.equal(got, torch.ops.mi355.gemm_nt(a, b, out_dtype, v))


@pytest.mark.parametrize("out_dtype", ["float16", "float32"])
@pytest.mark.parametrize("shape", [(4096, 4608, 256), (4352, 4352, 384), (8192, 8704, 512), (8192, 16384, 1152), (512, 256, 4096)])
def test_gemm_stream_tile_walk(dev, shape, out_dtype):
    """The streamed kernel launched with one workgroup per CU: every workgroup walks several tiles as one slab sequence
    (loads past a tile's end fetch the next tile's first slabs, a tile's first slab runs without load waits, the
    epilogue uses the part of LDS the next loads reach last, the first MFMA on each accumulator takes a zero addend).
    More tiles than CUs with a ragged last round, the minimum of four slabs, slab counts 2 and 0 mod 4 and 0, 1, 2 mod 3,
    up to nine tiles per workgroup, fewer tiles than CUs -- whole matrix bit-identical to the same kernel launched one
    workgroup per tile, and against the independent generic kernel."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"gemm streamed walk {shape} {out_dtype}")
    names = ita._lib.variants("gemm_f16_nt")
    walk, plain = names.index("stream_256x256x64_w2x2_walk"), names.index("stream_256x256x64_w2x2")
    a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K)]
    got = torch.ops.mi355.gemm_nt(a, b, out_dtype, walk)
    assert torch.equal(got, torch.ops.mi355.gemm_nt(a, b, out_dtype, plain))
    assert torch.equal(got, torch.ops.mi355.gemm_nt(a, b, out_dtype, walk))
    ref = torch.ops.mi355.gemm_nt(a, b, out_dtype, len(names) - 1)
    torch.testing.assert_close(got.float(), ref.float(), rtol=1e-3, atol=1e-3)


def test_gemm_stream_contract(dev):
    import iree_turbine_amd as ita

    names = ita._lib.variants("gemm_f16_nt")
    v = names.index("stream_256x256x64_w2x2")
    a = torch.zeros(256, 192, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a, a, "float16", v)  # K = 192 is not a whole number of slab pairs


@pytest.mark.parametrize("out_dtype", ["float16", "float32"])
@pytest.mark.parametrize("shape", [(2048, 10240, 512), (10240, 2048, 256), (768, 23296, 256), (2048, 8448, 256)])
@pytest.mark.parametrize("family", ["stream"])
def test_gemm_tail_split(dev, shape, out_dtype, family):
    """The streamed kernel with its sparse last round handed to the 128x128 kernel: a strip of tile columns
    (2048 x 10240: 64 of 320 tiles), a strip of tile rows (10240 x 2048), a remainder that is neither (runs
    unsplit) and the smallest strip (one tile column after a full round of 8 x 32) -- bit-identical to the
    unsplit kernel (both accumulate K in the same order), whole matrix against the generic kernel."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"gemm tail split {family} {shape} {out_dtype}")
    names = ita._lib.variants("gemm_f16_nt")
    v = next(i for i, n in enumerate(names) if n.startswith(family) and "tail" in n)
    staged = next(i for i, n in enumerate(names) if n.startswith(family) and "tail" not in n)
    a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K)]
    got = torch.ops.mi355.gemm_nt(a, b, out_dtype, v)
    assert torch.equal(got, torch.ops.mi355.gemm_nt(a, b, out_dtype, staged))
    ref = torch.ops.mi355.gemm_nt(a, b, out_dtype, len(names) - 1)
    torch.testing.assert_close(got.float(), ref.float(), rtol=1e-3, atol=1e-3)
    rows = torch.tensor([0, 255, M - 256, M - 1])
    exact = a[rows.to(dev)].float() @ b.float().t()
    torch.testing.assert_close(got[rows.to(dev)].float(), exact, rtol=RTOL, atol=ATOL)


def test_gemm_staged_contract(dev):
    import iree_turbine_amd as ita

    names = ita._lib.variants("gemm_f16_nt")
    v = next(i for i, n in enumerate(names) if n.startswith("staged"))
    a = torch.zeros(256, 192, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a, a, "float16", v)  # K = 192 is not a whole number of slab pairs
    a = torch.zeros(256, 128, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a, a, "float16", v)  # fewer than four slabs


@pytest.mark.parametrize("shape", [(32, 12, 64), (256, 512, 384), (100, 70, 72)])
@pytest.mark.parametrize("out_dtype", ["float16", "float32", "bfloat16"])
def test_gemm_autograd(dev, shape, out_dtype):
    """Gradients of the op against torch's own for C = A . B^T (the reference checks its GEMM backward formulas the
    same way, tests/kernel/boo/op_exports/gemm_backward_test.py:17-83), fp32 reference on the CPU."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs

    M, N, K = shape
    announce(f"gemm autograd {shape} {out_dtype}")
    in_dtype = torch.bfloat16 if out_dtype == "bfloat16" else torch.float16
    a, b = inputs.gemm_inputs(M, N, K, seed=1, dtype=in_dtype)
    w = torch.randn(M, N, generator=torch.Generator().manual_seed(2)) * 0.1
    ar, br = a.float().requires_grad_(True), b.float().requires_grad_(True)
    ((ar @ br.t()) * w).sum().backward()
    ad, bd = a.to(dev).requires_grad_(True), b.to(dev).requires_grad_(True)
    c = torch.ops.mi355.gemm_nt(ad, bd, out_dtype, -1)
    (c.float() * w.to(dev)).sum().backward()
    assert ad.grad.dtype == in_dtype and bd.grad.dtype == in_dtype
    tol = 3e-2 if in_dtype == torch.bfloat16 else RTOL  # bf16 keeps 8 bits: the upstream gradient and the result are rounded to it
    torch.testing.assert_close(ad.grad.float().cpu(), ar.grad, rtol=tol, atol=tol)
    torch.testing.assert_close(bd.grad.float().cpu(), br.grad, rtol=tol, atol=tol)
    # only one operand needs a gradient
    ad2 = a.to(dev).requires_grad_(True)
    torch.ops.mi355.gemm_nt(ad2, b.to(dev), out_dtype, -1).float().sum().backward()
    torch.testing.assert_close(ad2.grad.float().cpu(), b.float().sum(dim=0).expand(M, K), rtol=tol, atol=tol)


def test_gemm_output_beyond_4_gib(dev):
    """A 49152 x 49152 fp16 result is 4.5 GiB: row offsets into C pass 2^32 bytes.  Sampled rows (the first, two
    either side of the 4 GiB line, the last tile's) against an fp32 product, for the kernels the automatic choice
    can reach and the any-shape kernel."""
    import iree_turbine_amd as ita

    M = N = 49152
    K = 256
    names = ita._lib.variants("gemm_f16_nt")
    gen = torch.Generator(device="cpu").manual_seed(5)
    a = (torch.randn(M, K, generator=gen) * 0.1).half().to(dev)
    b = (torch.randn(N, K, generator=gen) * 0.1).half().to(dev)
    rows = torch.tensor([0, 1000, 43690, 43691, M - 257, M - 1], device=dev)
    ref = a[rows].float() @ b.float().t()
    tails = [i for i, n in enumerate(names) if "tail" in n]
    for variant in (-1, *tails, 0, names.index("pipelined_128x128x64_w2x2"), len(names) - 1):
        announce(f"gemm {M}x{N}x{K} float16 variant={variant} (C beyond 4 GiB)")
        c = torch.ops.mi355.gemm_nt(a, b, "float16", variant)
        torch.testing.assert_close(c[rows].float(), ref, rtol=RTOL, atol=ATOL)
        del c


BF16_SHAPES = [(1024, 1024, 1024), (256, 256, 256), (512, 768, 384), (2048, 10240, 512), (100, 70, 72), (33, 129, 40)]


@pytest.mark.parametrize("out_dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("shape", BF16_SHAPES)
def test_gemm_bf16_every_variant(dev, shape, out_dtype):
    """bf16 operands through every kernel variant that accepts the shape (same tiles, other MFMA instruction and
    epilogue conversion): whole matrix against the fp32 product of the same bf16 values.  fp32 results to 1e-3 of
    the largest entry (accumulation order only); bf16 results must be the fp32 result of the same variant rounded
    to nearest even."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    a, b = inputs.gemm_inputs(M, N, K, seed=21, dtype=torch.bfloat16)
    ref = a.float() @ b.float().t()
    a, b = a.to(dev), b.to(dev)
    names = ita._lib.variants("gemm_f16_nt")
    ran = 0
    for variant in [-1] + list(range(len(names))):
        announce(f"gemm_nt bf16 {shape} out={out_dtype} variant={variant}")
        try:
            c = torch.ops.mi355.gemm_nt(a, b, out_dtype, variant)
        except ValueError:
            continue  # the variant's tile does not divide this shape
        ran += 1
        assert c.dtype == getattr(torch, out_dtype)
        if out_dtype == "float32":
            torch.testing.assert_close(c.cpu(), ref, rtol=1e-3, atol=1e-3 * ref.abs().max().item())
        else:
            c32 = torch.ops.mi355.gemm_nt(a, b, "float32", variant)
            assert torch.equal(c, c32.bfloat16()), names[variant]
            torch.testing.assert_close(c.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    assert ran >= 2  # at least the automatic choice and the any-shape kernel


def test_gemm_bf16_full_size(dev):
    """8192^3 in bf16: sampled rows against the fp32 product, and the same launch twice is bit-identical."""
    from oracle import inputs

    M = N = K = 8192
    announce("gemm_nt bf16 8192^3")
    a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K, dtype=torch.bfloat16)]
    c = torch.ops.mi355.gemm_nt(a, b, "bfloat16", -1)
    rows = torch.tensor([0, 255, 4097, M - 1], device=dev)
    torch.testing.assert_close(c[rows].float(), a[rows].float() @ b.float().t(), rtol=RTOL, atol=ATOL)
    assert torch.equal(c, torch.ops.mi355.gemm_nt(a, b, "bfloat16", -1))


def test_gemm_dtype_contract(dev):
    a16 = torch.zeros(64, 64, dtype=torch.float16, device=dev)
    abf = torch.zeros(64, 64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a16, abf, "float32", -1)  # mixed operand formats
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(abf, abf, "float16", -1)  # 16-bit output is the operands' own format
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a16, a16, "bfloat16", -1)


@pytest.mark.parametrize("shape,dtype,out_dtype", [((3000, 5000, 4104), torch.float16, "float16"),
                                                   ((1100, 4200, 2056), torch.bfloat16, "float32"),
                                                   ((2304, 4096, 4100), torch.float16, "float32"),
                                                   ((2100, 4096, 4096), torch.bfloat16, "bfloat16"),
                                                   ((4100, 4096, 1024), torch.float16, "float16"),
                                                   ((2432, 4096, 2048), torch.float16, "float32"),
                                                   ((5000, 2048, 512), torch.bfloat16, "bfloat16")])
def test_gemm_large_ragged_shapes_take_the_padded_path(dev, shape, dtype, out_dtype):
    """Large products whose sizes are not tile multiples run on the tiled kernels: over zero-padded copies when N or K is
    ragged (only the ragged operands are copied), as a multiple of 256 rows and a remainder in two launches on row
    ranges of the caller's tensors when only M is (2100 = 2048 + 52, 4100 = 4096 + 4, 2432 = 2304 + 128 rows): the
    result must be what the bounds-checked kernel gives on the original operands, and the caller's tensors stay
    untouched."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"gemm ragged {shape} {dtype} -> {out_dtype}")
    a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K, seed=31, dtype=dtype)]
    a0, b0 = a.clone(), b.clone()
    names = ita._lib.variants("gemm_f16_nt")
    got = torch.ops.mi355.gemm_nt(a, b, out_dtype, -1)
    assert got.shape == (M, N) and got.is_contiguous()
    ref = torch.ops.mi355.gemm_nt(a, b, out_dtype, len(names) - 1)
    # another kernel adds up in another order: fp32 results agree to 1e-3, 16-bit results to one step of their format
    tol = 1e-3 if out_dtype == "float32" else (2.0 ** -7 if out_dtype == "bfloat16" else 2.0 ** -10)
    torch.testing.assert_close(got.float(), ref.float(), rtol=tol, atol=1e-3)
    rows = torch.tensor([0, M // 2, M - 1], device=dev)
    torch.testing.assert_close(got[rows].float(), a[rows].float() @ b.float().t(), rtol=RTOL, atol=ATOL)
    assert torch.equal(a, a0) and torch.equal(b, b0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(16, 8192, 8192), (1, 4096, 4096), (32, 2048, 192), (7, 256, 64), (32, 32, 448), (5, 64, 1088),
                                   (20, 4096, 14336), (31, 96, 8256), (64, 4096, 4096), (33, 2048, 1024), (50, 64, 320),
                                   (64, 32, 64), (40, 96, 448), (48, 2048, 8256), (64, 8192, 8192), (57, 4096, 1088),
                                   (65, 2048, 1024), (100, 4096, 2048), (128, 64, 320), (127, 2048, 8192), (96, 32, 64)])
def test_gemm_skinny_m(dev, shape, dtype):
    """The weight-streaming kernels for M <= 128 (33 to 64 rows take the kernel with two row blocks and eight waves, 65 to 128
    rows four row blocks and four waves; the automatic choice takes them up to 64 rows and for ragged M beyond): one to 128 rows, one K
    segment per wave and fewer segments than waves, odd segment counts (the double buffer ends on either half), several
    segments per wave, more workgroups per XCD than segments per wave (the rotated start wraps); fp32 result against the
    fp32 product of the same values, 16-bit result = the fp32 result rounded, launches repeat bit for bit, and
    decode-shaped products take this kernel by themselves."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    names = ita._lib.variants("gemm_f16_nt")
    sk = next(i for i, n in enumerate(names) if n.startswith("skinny"))
    own = str(dtype).removeprefix("torch.")
    announce(f"gemm skinny {shape} {own} variant={sk}")
    a, b = inputs.gemm_inputs(M, N, K, seed=13, dtype=dtype)
    ref = a.float() @ b.float().t()
    a, b = a.to(dev), b.to(dev)
    c32 = torch.ops.mi355.gemm_nt(a, b, "float32", sk)
    torch.testing.assert_close(c32.cpu(), ref, rtol=1e-3, atol=1e-3 * max(1.0, ref.abs().max().item()))
    c16 = torch.ops.mi355.gemm_nt(a, b, own, sk)
    assert torch.equal(c16, c32.to(dtype))
    assert torch.equal(c32, torch.ops.mi355.gemm_nt(a, b, "float32", sk))
    if N >= 2048 and K >= 512 and (M <= 64 or M % 64):
        assert torch.equal(c32, torch.ops.mi355.gemm_nt(a, b, "float32", -1))


def test_gemm_skinny_contract(dev):
    import iree_turbine_amd as ita

    names = ita._lib.variants("gemm_f16_nt")
    sk = next(i for i, n in enumerate(names) if n.startswith("skinny"))
    a = torch.zeros(129, 64, dtype=torch.float16, device=dev)
    b = torch.zeros(64, 64, dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a, b, "float32", sk)  # 129 rows
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a[:8], b[:48], "float32", sk)  # N = 48 is not whole 32-row tiles
    with pytest.raises(ValueError):
        torch.ops.mi355.gemm_nt(a[:8, :32].contiguous(), b[:, :32].contiguous(), "float32", sk)  # K = 32 < one segment


@pytest.mark.parametrize("out_dtype", ["float16", "float32"])
@pytest.mark.parametrize("shape", [(2048, 10240, 8192), (10240, 2048, 6144), (2048, 4096, 8192), (2048, 1280, 4096), (256, 2048, 8192),
                                   (384, 640, 8192), (256, 256, 8192), (128, 128, 2048), (64, 1024, 4096), (512, 512, 4096),
                                   (128, 2112, 4096), (128, 4160, 8192), (256, 4224, 32768), (128, 2432, 32768)])
def test_gemm_k_split_with_workspace(dev, shape, out_dtype):
    """The workspace entry point through the C ABI: a strip of tile columns (2048 x 10240: the last 64 of 320 tiles, four
    K ranges), a strip of tile rows (four ranges of 1536), a whole product of 128 tiles of 256x256 (two ranges), 160 tiles
    of 128x128 in two ranges, and small products that split on 64x64 tiles (two, four and eight ranges; one shape no
    multiple of 128, one a single tile, one a single tile row), on 128x64 tiles (four and two ranges) and on 128x128
    tiles (K = 32768: two and eight ranges) -- the whole matrix against the plain entry point (same products, other
    summation order), sampled rows against an fp32 product; a workspace one byte short or absent runs exactly as the plain entry point does."""
    from iree_turbine_amd import _lib
    from oracle import inputs

    M, N, K = shape
    announce(f"gemm K split {shape} {out_dtype}")
    lib = _lib.load()
    a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K)]
    dt = getattr(torch, out_dtype)
    need = lib.mi355_gemm_nt_workspace_bytes(M, N, K)
    assert need > 0 and need % 1024 == 0
    ws = torch.empty(need // 4, dtype=torch.float32, device=dev)
    stream = _lib.current_stream_ptr(dev)

    def run(ws_ptr, ws_bytes):
        c = torch.full((M, N), float("nan"), dtype=dt, device=dev)
        rc = lib.mi355_gemm_f16_nt_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, _lib.dtype_code(dt), -1, ws_ptr, ws_bytes, stream)
        _lib.check(rc, "gemm_f16_nt_ws")
        return c

    plain = torch.empty((M, N), dtype=dt, device=dev)
    _lib.check(lib.mi355_gemm_f16_nt(a.data_ptr(), b.data_ptr(), plain.data_ptr(), M, N, K, _lib.dtype_code(dt), -1, stream), "gemm_f16_nt")
    split = run(ws.data_ptr(), need)
    assert torch.equal(split, run(ws.data_ptr(), need))  # launches repeat bit for bit (the workspace is scratch)
    assert not torch.equal(split, plain) or out_dtype == "float16"  # another summation order: fp32 sums differ in the last bits
    tol = dict(rtol=1e-4, atol=1e-4) if out_dtype == "float32" else dict(rtol=2e-3, atol=1e-3)
    torch.testing.assert_close(split.float(), plain.float(), **tol)
    rows = torch.tensor([0, min(255, M - 1), max(M - 256, 0), M - 1], device=dev)  # sampled rows, inside the matrix for the small shapes too
    exact = a[rows].float() @ b.float().t()
    torch.testing.assert_close(split[rows].float(), exact, rtol=RTOL, atol=ATOL)
    assert torch.equal(run(ws.data_ptr(), need - 1), plain)
    assert torch.equal(run(None, 0), plain)


def test_gemm_k_split_through_the_op(dev):
    """torch.ops.mi355.gemm_nt allocates the workspace the library asks for: a small product (bf16 operands) and
    the benchmark shape with the sparse last round against the oracle's rows; shapes that take no split ask for none."""
    from iree_turbine_amd import _lib
    from oracle import inputs

    lib = _lib.load()
    assert lib.mi355_gemm_nt_workspace_bytes(8192, 8192, 8192) == 0
    assert lib.mi355_gemm_nt_workspace_bytes(4096, 4096, 4096) == 0
    assert lib.mi355_gemm_nt_workspace_bytes(16, 8192, 8192) == 0
    assert lib.mi355_gemm_nt_workspace_bytes(2048, 10240, 4096) == 0  # K too short for 64 tiles' partial products to pay
    assert lib.mi355_gemm_nt_workspace_bytes(2048, 4096, 8192) == 2 * 2048 * 4096 * 4
    assert lib.mi355_gemm_nt_workspace_bytes(2048, 10240, 8192) == 4 * 2048 * 2048 * 4
    for (M, N, K), dtype in (((512, 2048, 8192), torch.bfloat16), ((2048, 10240, 8192), torch.float16)):
        announce(f"gemm K split through the op {(M, N, K)} {dtype}")
        a, b = [t.to(dev) for t in inputs.gemm_inputs(M, N, K, dtype=dtype)]
        c = torch.ops.mi355.gemm_nt(a, b, "float32", -1)
        rows = torch.tensor([0, 300, M - 1], device=dev)
        torch.testing.assert_close(c[rows], a[rows].float() @ b.float().t(), rtol=1e-3, atol=1e-3)
        cols = torch.tensor([0, N - 2048, N - 1], device=dev)
        torch.testing.assert_close(c[:, cols], a.float() @ b[cols].float().t(), rtol=1e-3, atol=1e-3)
