"""GPU parity: MXFP4 dequantisation (bit-exact) and block-scaled GEMM (<= 1e-2 relative) through the C ABI."""

import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

REL = 1e-2  # the contract: GEMM within 1e-2 relative of an fp32 matmul on the dequantised operands


def _rel_err(c: torch.Tensor, ref: torch.Tensor) -> float:
    return ((c.double() - ref.double()).norm() / ref.double().norm()).item()


def test_dequant_exhaustive_bit_exact(dev):
    """All 16 codes x all 256 scale bytes, in both nibble positions, bit for bit (NaN for 0xFF)."""
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp4 as om

    announce("mxfp4 dequant exhaustive")
    rows, K = 256, 64
    k = np.arange(K)
    elem_codes = np.where(k < 32, k % 16, (k + 1) % 16).astype(np.uint8)  # every code in both nibble positions
    packed = torch.from_numpy(np.ascontiguousarray(np.broadcast_to(om.pack_codes(elem_codes[None, :]), (rows, K // 2))))
    scales = torch.arange(256, dtype=torch.int32).to(torch.uint8).reshape(rows, 1).repeat(1, 2)
    out = torch.ops.mi355.mxfp4_dequant(packed.to(dev), scales.to(dev)).cpu().numpy()
    ref = om.mxfp4_dequant_ref(packed, scales)
    assert out.dtype == np.float32 and out.shape == ref.shape
    assert np.array_equal(out.view(np.uint32)[:255], ref.view(np.uint32)[:255])
    assert np.isnan(out[255]).all() and np.isnan(ref[255]).all()


def test_dequant_random_bit_exact(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, mxfp4 as om

    announce("mxfp4 dequant random")
    a, asc, _, _ = inputs.mxfp4_inputs(96, 8, 1024, seed=2)
    out = torch.ops.mi355.mxfp4_dequant(a.to(dev), asc.to(dev)).cpu().numpy()
    assert np.array_equal(out.view(np.uint32), om.mxfp4_dequant_ref(a, asc).view(np.uint32))


@pytest.mark.parametrize("variant", [-1, 0, 1, 2, 4, 5, 6, 7, 8])
def test_mxfp4_gemm_variants(dev, variant):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, mxfp4 as om

    M, N, K = 512, 768, 1024
    announce(f"mxfp4_gemm M={M} N={N} K={K} variant={variant}")
    a, asc, b, bsc = inputs.mxfp4_inputs(M, N, K, seed=7)
    ref = om.mxfp4_gemm_ref(a, asc, b, bsc)
    c32 = torch.ops.mi355.mxfp4_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "float32", variant).cpu()
    assert _rel_err(c32, ref) < 1e-5
    c16 = torch.ops.mi355.mxfp4_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "bfloat16", variant).cpu()
    assert _rel_err(c16, ref) < REL
    torch.testing.assert_close(c16.float(), ref, rtol=REL, atol=REL * ref.abs().max().item())
    assert torch.equal(c16, c32.bfloat16())  # the bf16 epilogue is round-to-nearest-even of the fp32 result


@pytest.mark.parametrize("shape", [(32, 256, 512), (1, 1, 32), (33, 65, 96), (32, 8192, 2048), (100, 40, 1056)])
def test_mxfp4_gemm_ragged(dev, shape):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, mxfp4 as om

    M, N, K = shape
    announce(f"mxfp4_gemm ragged {shape}")
    a, asc, b, bsc = inputs.mxfp4_inputs(M, N, K, seed=13)
    ref = om.mxfp4_gemm_ref(a, asc, b, bsc)
    c = torch.ops.mi355.mxfp4_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "float32", -1).cpu()
    assert _rel_err(c, ref) < 1e-5


@pytest.mark.parametrize("shape", [(32, 256, 512), (1, 64, 256), (7, 96, 2048), (32, 8192, 8192), (20, 160, 16384), (32, 64, 8192 + 256)])
@pytest.mark.parametrize("variant", [3, 8])
def test_mxfp4_skinny_vs_generic(dev, shape, variant):
    """The weight-streaming kernel (variant 3) and the any-shape kernel (variant 8) on skinny shapes."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, mxfp4 as om

    M, N, K = shape
    announce(f"mxfp4_gemm skinny {shape} variant={variant}")
    a, asc, b, bsc = inputs.mxfp4_inputs(M, N, K, seed=17)
    ref = om.mxfp4_gemm_ref(a, asc, b, bsc)
    c = torch.ops.mi355.mxfp4_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "float32", variant).cpu()
    assert _rel_err(c, ref) < 1e-5
    c16 = torch.ops.mi355.mxfp4_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "bfloat16", variant).cpu()
    assert torch.equal(c16, c.bfloat16())


def test_mxfp4_one_hot_nibble_order_and_scale_block(dev):
    """A single non-zero code at element k of A picks out B[:, k]: pins the nibble order (even k = low
    nibble) and which 32-element block a scale byte belongs to."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, mxfp4 as om

    announce("mxfp4 one-hot")
    M, N, K = 32, 64, 256
    _, _, b, bsc = inputs.mxfp4_inputs(M, N, K, seed=5)
    db = om.mxfp4_dequant_ref(b, bsc)
    for k in (0, 1, 31, 32, 63, 130, 255):
        a = torch.zeros(M, K // 2, dtype=torch.uint8)
        a[3, k // 2] = 0x2 << (4 * (k % 2))  # code 2 = 1.0
        asc = torch.full((M, K // 32), 127, dtype=torch.uint8)
        asc[3, k // 32] = 130  # x8 on that block only
        c = torch.ops.mi355.mxfp4_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "float32", -1).cpu().numpy()
        assert np.array_equal(c[3], 8.0 * db[:, k]), k
        assert not c[np.arange(M) != 3].any()


def test_mxfp4_exact_cases(dev):
    """Unit scales and codes in {0, 1, 2, 4}: small-integer sums, exact.  Then +1 on every A scale byte
    doubles the result exactly."""
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp4 as om

    announce("mxfp4 exact cases")
    M, N, K = 256, 256, 512
    g = torch.Generator().manual_seed(3)
    pick = torch.tensor([0, 2, 4, 6], dtype=torch.uint8)  # codes of 0, 1, 2, 4
    ca = pick[torch.randint(0, 4, (M, K), generator=g)]
    cb = pick[torch.randint(0, 4, (N, K), generator=g)]
    a = torch.from_numpy(om.pack_codes(ca.numpy()))
    b = torch.from_numpy(om.pack_codes(cb.numpy()))
    one = torch.full((M, K // 32), 127, dtype=torch.uint8)
    ref = om.mxfp4_gemm_ref(a, one, b, one)
    c = torch.ops.mi355.mxfp4_gemm(a.to(dev), one.to(dev), b.to(dev), one.to(dev), "float32", -1).cpu()
    assert torch.equal(c, ref)
    c2 = torch.ops.mi355.mxfp4_gemm(a.to(dev), (one + 1).to(dev), b.to(dev), one.to(dev), "float32", -1).cpu()
    assert torch.equal(c2, 2 * c)


@pytest.mark.parametrize("shape", [(4096, 8192, 8192), (32, 8192, 8192)])
def test_mxfp4_full_size(dev, shape):
    """Benchmark shapes: sampled rows and columns against the oracle."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, mxfp4 as om

    M, N, K = shape
    announce(f"mxfp4 full size {shape}")
    a, asc, b, bsc = inputs.mxfp4_inputs(M, N, K)
    c = torch.ops.mi355.mxfp4_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "bfloat16", -1)
    rows = torch.tensor(sorted({0, 1, 31, M // 2, M - 1}))
    cols = torch.tensor([0, 255, 256, N // 2 + 5, N - 1])
    ref_r = om.mxfp4_gemm_ref(a[rows], asc[rows], b, bsc)
    got_r = c[rows.to(dev)].float().cpu()
    assert _rel_err(got_r, ref_r) < REL
    ref_c = om.mxfp4_gemm_ref(a, asc, b[cols], bsc[cols])
    got_c = c[:, cols.to(dev)].float().cpu()
    assert _rel_err(got_c, ref_c) < REL
    # element by element as well, so that one bad tile column cannot hide inside a norm: bf16 rounding is 2^-9
    # relative, and an element that cancels to near zero is held to 1e-2 of the largest magnitude instead
    torch.testing.assert_close(got_r, ref_r, rtol=REL, atol=REL * ref_r.abs().max().item())
    torch.testing.assert_close(got_c, ref_c, rtol=REL, atol=REL * ref_c.abs().max().item())


@pytest.mark.parametrize("shape", [(4096, 8192, 8192), (32, 8192, 8192)])
def test_mxfp4_full_size_repeatable(dev, shape):
    """Whole-matrix checks at benchmark sizes: each variant that accepts the shape is bit-identical across
    launches and agrees with the simple generic kernel."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"mxfp4 repeatability {shape}")
    a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp4_inputs(M, N, K)]
    names = ita._lib.variants("mxfp4_gemm")
    generic = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, "float32", len(names) - 1)
    ran = 0
    for variant in range(len(names) - 1):
        try:
            first = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, "float32", variant)
        except ValueError:
            continue  # the variant's tile does not divide this shape
        ran += 1
        for _ in range(2):
            assert torch.equal(first, torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, "float32", variant)), names[variant]
        assert _rel_err(first, generic) < 1e-5, names[variant]
    assert ran >= 1


@pytest.mark.parametrize("shape", [(128, 128, 1024), (64, 64, 1024), (256, 256, 2048), (192, 320, 3072), (384, 640, 5120), (1024, 1024, 8192),
                                   (128, 8192, 8192), (2048, 2048, 2048), (2048, 2176, 1024), (1152, 1152, 4096), (64, 28672, 1024)])
@pytest.mark.parametrize("out_dtype", ["bfloat16", "float32"])
def test_mxfp4_slab_form(dev, shape, out_dtype):
    """The tiled kernel's slab form (four data stages, a whole slab's fragments and scale dwords in one of two register
    sets, scale groups of four slabs riding with every fourth trip): one tile and one scale group (the minimum K), two,
    three, five and eight groups, shapes that are no multiple of 128, 256 tiles of either shape, and 272 tiles of
    128x128 (the k-step form) -- the 64x64 and 128x128 tiles by index and the automatic choice, whole matrix against
    the independent generic kernel, launches repeat bit for bit."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"mxfp4 slab form {shape} {out_dtype}")
    names = ita._lib.variants("mxfp4_gemm")
    a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp4_inputs(M, N, K, seed=M + N + K)]
    ref = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, len(names) - 1)
    todo = [-1, names.index("tiled_64x64x256_w2x2")] + ([names.index("tiled_128x128x256_w2x2")] if M % 128 == 0 and N % 128 == 0 else [])
    for v in todo:
        got = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, v)
        if out_dtype == "float32":
            assert _rel_err(got, ref) < 1e-5, v
        else:
            g32, r32 = got.float(), ref.float()
            assert _rel_err(g32, r32) < 1e-3, v
            assert ((g32 - r32).abs() <= r32.abs() * 2 ** -7 + 1e-5 * r32.abs().max()).all(), v
        assert torch.equal(got, torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, v)), v


@pytest.mark.parametrize("shape", [(33, 64, 1024), (65, 128, 2048), (100, 8192, 1024), (127, 64, 3072), (200, 2048, 4096), (1000, 1024, 1024),
                                   (129, 4160, 1024), (2100, 4096, 1024), (4100, 2048, 2048), (540, 8192, 1024)])
@pytest.mark.parametrize("out_dtype", ["bfloat16", "float32"])
def test_mxfp4_ragged_rows(dev, shape, out_dtype):
    """Any number of rows beyond the weight-streaming kernel's 32 against N % 64 == 0 and K % 1024 == 0: the 64x64 tile
    with its last tile row cut (codes and scales of A read from row min(row, M - 1), stores stop at M), and from 512
    rows the multiple of 256 and the remainder as two products (2048 + 52, 4096 + 4, 512 + 28 rows) -- whole matrix
    against the bounds-checked kernel, the rows behind the result untouched, launches repeat bit for bit."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"mxfp4 ragged rows {shape} {out_dtype}")
    names = ita._lib.variants("mxfp4_gemm")
    a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp4_inputs(M, N, K, seed=M + N + K)]
    ref = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, len(names) - 1)
    odt = getattr(torch, out_dtype)
    full = torch.full((M + 70, N), float("nan"), dtype=odt, device=dev)
    got = full[:M]
    ita.launch.mxfp4_gemm_out(a, asc, b, bsc, got, -1)
    if out_dtype == "float32":
        assert _rel_err(got, ref) < 1e-5
    else:
        g32, r32 = got.float(), ref.float()
        assert _rel_err(g32, r32) < 1e-3
        assert ((g32 - r32).abs() <= r32.abs() * 2 ** -7 + 1e-5 * r32.abs().max()).all()
    assert torch.isnan(full[M:]).all()
    again = torch.empty_like(got)
    ita.launch.mxfp4_gemm_out(a, asc, b, bsc, again, -1)
    assert torch.equal(got, again)


@pytest.mark.parametrize("shape", [(4352, 4352, 1024), (4096, 4608, 1536), (512, 256, 8192)])
@pytest.mark.parametrize("out_dtype", ["bfloat16", "float32"])
def test_mxfp4_persistent_tile_walk(dev, shape, out_dtype):
    """The persistent kernel walks several tiles per workgroup as one slab sequence: more tiles than CUs,
    tile counts that are not multiples of 8 or of the grid, an odd number of scale groups per tile (the
    scale buffer parity flips between tiles), the minimum K, fewer tiles than CUs -- whole matrix against
    the independent generic kernel."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"mxfp4 persistent walk {shape} {out_dtype}")
    names = ita._lib.variants("mxfp4_gemm")
    assert names[0].startswith("persistent")
    a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp4_inputs(M, N, K)]
    got = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, 0)
    ref = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, len(names) - 1)
    if out_dtype == "float32":
        assert _rel_err(got, ref) < 1e-5
    else:
        # both round the same fp32 sums (up to summation order) to bf16: at most one bf16 step apart,
        # plus the summation-order noise of sums that cancel to nearly nothing
        g32, r32 = got.float(), ref.float()
        assert _rel_err(g32, r32) < 1e-3
        assert ((g32 - r32).abs() <= r32.abs() * 2 ** -7 + 1e-5 * r32.abs().max()).all()


@pytest.mark.parametrize("shape", [(256, 256, 1024), (512, 768, 1536), (4352, 4352, 1024), (4096, 4608, 2560), (8192, 8704, 1024),
                                   (256, 512, 8192)])
@pytest.mark.parametrize("out_dtype", ["bfloat16", "float32"])
def test_mxfp4_stream_tile_walk(dev, shape, out_dtype):
    """The streamed kernel: B in a ring of five half buffers (slab counts 4, 6, 10, 32: the ring position at a tile's end takes
    every value), scale groups of two slabs (even and odd numbers of groups per tile: the
    scale buffer parity flips between tiles), more tiles than CUs with a ragged last round, up to five tiles per
    workgroup, fewer tiles than CUs -- the walk bit-identical to the same kernel launched one workgroup per tile,
    whole matrix against the independent generic kernel, launches repeat bit for bit."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"mxfp4 streamed walk {shape} {out_dtype}")
    names = ita._lib.variants("mxfp4_gemm")
    walk, plain = names.index("stream_256x256x256_w2x2_walk"), names.index("stream_256x256x256_w2x2")
    a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp4_inputs(M, N, K)]
    got = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, walk)
    assert torch.equal(got, torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, plain))
    assert torch.equal(got, torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, walk))
    ref = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, len(names) - 1)
    if out_dtype == "float32":
        assert _rel_err(got, ref) < 1e-5
    else:
        g32, r32 = got.float(), ref.float()
        assert _rel_err(g32, r32) < 1e-3
        assert ((g32 - r32).abs() <= r32.abs() * 2 ** -7 + 1e-5 * r32.abs().max()).all()


def test_mxfp4_contract_errors(dev):
    import iree_turbine_amd  # noqa: F401

    a = torch.zeros(32, 16, dtype=torch.uint8, device=dev)
    s = torch.full((32, 1), 127, dtype=torch.uint8, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp4_gemm(a, s, a[:, :8], s, "bfloat16", -1)
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp4_gemm(a, s[:, :0], a, s, "bfloat16", -1)
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp4_gemm(a, s, a, s, "float16", -1)


@pytest.mark.parametrize("shape", [(256, 256, 1024), (512, 768, 1536), (4352, 4352, 1024), (256, 512, 8192)])
@pytest.mark.parametrize("out_dtype", ["bfloat16", "float32"])
def test_mxfp4_staged_slab_rotation(dev, shape, out_dtype):
    """The register-staged kernel keeps three slabs and two scale groups in flight: the minimum of four slabs,
    odd and even numbers of scale groups (the scale buffer parity), a ragged tile grid larger than the chip
    and a long K -- whole matrix against the independent generic kernel."""
    import iree_turbine_amd as ita
    from oracle import inputs

    M, N, K = shape
    announce(f"mxfp4 staged {shape} {out_dtype}")
    names = ita._lib.variants("mxfp4_gemm")
    v = next(i for i, n in enumerate(names) if n.startswith("staged"))
    a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp4_inputs(M, N, K)]
    got = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, v)
    ref = torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, len(names) - 1)
    if out_dtype == "float32":
        assert _rel_err(got, ref) < 1e-5
    else:
        g32, r32 = got.float(), ref.float()
        assert _rel_err(g32, r32) < 1e-3
        assert ((g32 - r32).abs() <= r32.abs() * 2 ** -7 + 1e-5 * r32.abs().max()).all()
    assert torch.equal(got, torch.ops.mi355.mxfp4_gemm(a, asc, b, bsc, out_dtype, v))
