"""GPU parity: block-scaled MXFP8 GEMM through the C ABI vs the CPU oracle (table dequantise + fp32 matmul).
Contract as for MXFP4: the decode is exact (every product of two fp8 values and two power-of-two scales is exact
in fp32), the GEMM within 1e-2 relative of the fp32 matmul on the dequantised operands."""

import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

REL = 1e-2
# The matrix unit adds the products of one 16-element lane group in fixed point, aligned to the largest of them
# with 13 bits below it (measured: 2^16 + 2^3 is kept, 2^16 + 2^2 is not); sums across groups and with the
# accumulator are full fp32.  With E4M3's 2^17 range of magnitudes that shows as ~1e-4 of the largest output;
# a single product per group is exact.
HW_SUM = 5e-4


def _rel_err(got, ref):
    return ((got.double() - ref.double()).abs().max() / ref.double().abs().max()).item()


def test_mxfp8_decode_exhaustive(dev):
    """Every finite E4M3 code against the scale bytes 20..234, through the GEMM with a one-hot partner: the
    single product of each output cell is exact, so the result must equal the table bit for bit."""
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp8 as o8

    announce("mxfp8 decode exhaustive")
    K = 32
    codes = torch.arange(256, dtype=torch.uint8)
    finite = codes[(codes & 0x7F) != 0x7F]
    a = torch.zeros(len(finite), K, dtype=torch.uint8)
    a[:, 0] = finite
    b = torch.zeros(32, K, dtype=torch.uint8)
    b[:, 0] = 0x38  # 1.0
    bsc = torch.full((32, 1), 127, dtype=torch.uint8)
    # scale bytes 20..234: every product stays a normal fp32 number (the matrix unit's treatment of fp32
    # denormals is not part of the contract)
    for sc in range(20, 235):
        asc = torch.full((len(finite), 1), sc, dtype=torch.uint8)
        c = torch.ops.mi355.mxfp8_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "float32", -1).cpu()
        want = o8.mxfp8_dequant_ref(a, asc)[:, 0]
        assert np.array_equal(c[:, 0].numpy().view(np.uint32) & 0x7FFFFFFF, want.view(np.uint32) & 0x7FFFFFFF), sc
        nz = want != 0
        assert np.array_equal(np.signbit(c[:, 0].numpy())[nz], np.signbit(want)[nz]), sc


@pytest.mark.parametrize("variant", [-1, 0, 1, 2, 3, 4])
def test_mxfp8_gemm_variants(dev, variant):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, mxfp8 as o8

    M, N, K = 512, 768, 1024
    announce(f"mxfp8_gemm M={M} N={N} K={K} variant={variant}")
    a, asc, b, bsc = inputs.mxfp8_inputs(M, N, K, seed=7)
    ref = o8.mxfp8_gemm_ref(a, asc, b, bsc)
    c32 = torch.ops.mi355.mxfp8_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "float32", variant).cpu()
    assert _rel_err(c32, ref) < HW_SUM
    c16 = torch.ops.mi355.mxfp8_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "bfloat16", variant).cpu()
    assert _rel_err(c16, ref) < REL
    assert torch.equal(c16, c32.bfloat16())  # the bf16 epilogue is round-to-nearest-even of the fp32 result


@pytest.mark.parametrize("shape", [(1, 1, 32), (33, 70, 96), (100, 260, 160), (257, 255, 2048), (256, 256, 256), (512, 256, 768)])
def test_mxfp8_gemm_shapes(dev, shape):
    """Ragged shapes (generic kernel: odd numbers of scale blocks, partial tiles) and the smallest / odd slab
    counts of the tiled kernel."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, mxfp8 as o8

    M, N, K = shape
    announce(f"mxfp8_gemm shape {shape}")
    a, asc, b, bsc = inputs.mxfp8_inputs(M, N, K, seed=5)
    ref = o8.mxfp8_gemm_ref(a, asc, b, bsc)
    c = torch.ops.mi355.mxfp8_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "float32", -1).cpu()
    assert _rel_err(c, ref) < HW_SUM


def test_mxfp8_one_hot_layout(dev):
    """A single non-zero element at every k position of a 512-wide row: pins which byte of a lane's 32
    belongs to which k and which scale byte goes with which block (a swapped half or block shows up here)."""
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp8 as o8

    announce("mxfp8 one-hot layout")
    K = 512
    a = torch.zeros(K, K, dtype=torch.uint8)
    a[torch.arange(K), torch.arange(K)] = 0x38  # row i has 1.0 at k = i
    g = torch.Generator().manual_seed(1)
    asc = (120 + torch.randint(0, 15, (K, K // 32), generator=g)).to(torch.uint8)
    b = torch.randint(0, 256, (256, K), generator=g).to(torch.uint8)
    b = torch.where((b & 0x7F) == 0x7F, b - 1, b)
    bsc = (120 + torch.randint(0, 15, (256, K // 32), generator=g)).to(torch.uint8)
    for variant in (0, 1, 2):
        c = torch.ops.mi355.mxfp8_gemm(a.to(dev), asc.to(dev), b.to(dev), bsc.to(dev), "float32", variant).cpu()
        # C[i, n] = 2^(asc[i, i/32] - 127) * dq(B)[n, i]
        db = torch.from_numpy(o8.mxfp8_dequant_ref(b, bsc))
        sa = torch.from_numpy(o8.mxfp8_dequant_ref(a, asc))[torch.arange(K), torch.arange(K)]
        assert torch.equal(c, sa[:, None] * db.t()), variant


def test_mxfp8_full_size_cross_variant(dev):
    import iree_turbine_amd as ita
    from oracle import inputs, mxfp8 as o8

    M, N, K = 2048, 4096, 4096
    announce(f"mxfp8 full size {M}x{N}x{K}")
    a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp8_inputs(M, N, K)]
    tiled = torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, "float32", 0)
    assert torch.equal(tiled, torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, "float32", 0))
    generic = torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, "float32", 1)
    assert _rel_err(tiled, generic) < HW_SUM  # the two kernels pair blocks differently
    rows = torch.tensor([0, 255, 256, 1023, M - 1])
    ref = o8.mxfp8_gemm_ref(a[rows.to(dev)].cpu(), asc[rows.to(dev)].cpu(), b.cpu(), bsc.cpu())
    assert _rel_err(tiled[rows.to(dev)].cpu(), ref) < HW_SUM
    # the register-staged kernel feeds the same block pairs to the same instruction in the same order
    staged = torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, "float32", 2)
    assert torch.equal(staged, tiled)
    assert torch.equal(staged, torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, "float32", 2))
    # the streamed kernel takes a whole 128-element slab per instruction
    names = ita._lib.variants("mxfp8_gemm")
    stream = torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, "float32", names.index("stream_256x256x128_w2x2_walk"))
    assert _rel_err(stream, generic) < HW_SUM
    assert torch.equal(stream, torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, "float32", -1))  # the automatic choice at this size


@pytest.mark.parametrize("out_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(256, 256, 512), (512, 768, 768), (1024, 512, 1280), (2048, 10240, 512), (256, 512, 8192)])
def test_mxfp8_staged_slab_rotation(dev, shape, out_dtype):
    """The register-staged kernel keeps three slabs in flight in two register sets and passes scales through
    parity buffers per pair of slabs: the minimum of four slabs, slab-pair counts that are odd and even, a grid
    larger than the chip, a long K -- whole matrix bit-identical to the two-stage kernel, rows against fp32."""
    import iree_turbine_amd as ita
    from oracle import inputs, mxfp8 as o8

    M, N, K = shape
    announce(f"mxfp8 staged {shape} {out_dtype}")
    names = ita._lib.variants("mxfp8_gemm")
    v = next(i for i, n in enumerate(names) if n.startswith("staged"))
    a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp8_inputs(M, N, K, seed=3)]
    got = torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, out_dtype, v)
    assert torch.equal(got, torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, out_dtype, 0))
    assert torch.equal(got, torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, out_dtype, v))
    rows = torch.tensor([0, 127, 128, M - 1])
    ref = o8.mxfp8_gemm_ref(a[rows.to(dev)].cpu(), asc[rows.to(dev)].cpu(), b.cpu(), bsc.cpu())
    assert _rel_err(got[rows.to(dev)].float().cpu(), ref) < (HW_SUM if out_dtype == "float32" else REL)


@pytest.mark.parametrize("shape", [(256, 256, 1024), (512, 768, 1536), (4352, 4352, 1024), (4096, 4608, 2560), (8192, 8704, 1024),
                                   (256, 512, 8192)])
@pytest.mark.parametrize("out_dtype", ["bfloat16", "float32"])
def test_mxfp8_stream_tile_walk(dev, shape, out_dtype):
    """The streamed kernel: B in a ring of five half buffers (slab counts 8, 12, 20, 64: the ring position at a tile's
    end takes every value), scale groups of four slabs (even and odd numbers of groups per tile: the scale buffer
    parity flips between tiles), more tiles than CUs with a ragged last round, up to five tiles per workgroup, fewer
    tiles than CUs -- the walk bit-identical to the same kernel launched one workgroup per tile, whole matrix against
    the independent generic kernel, rows against the fp32 oracle, launches repeat bit for bit."""
    import iree_turbine_amd as ita
    from oracle import inputs, mxfp8 as o8

    M, N, K = shape
    announce(f"mxfp8 streamed walk {shape} {out_dtype}")
    names = ita._lib.variants("mxfp8_gemm")
    walk, plain = names.index("stream_256x256x128_w2x2_walk"), names.index("stream_256x256x128_w2x2")
    a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp8_inputs(M, N, K, seed=11)]
    got = torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, out_dtype, walk)
    assert torch.equal(got, torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, out_dtype, plain))
    assert torch.equal(got, torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, out_dtype, walk))
    ref = torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, out_dtype, names.index("generic_32x128"))
    if out_dtype == "float32":
        assert _rel_err(got, ref) < HW_SUM
    else:
        g32, r32 = got.float(), ref.float()
        assert _rel_err(g32, r32) < REL
        assert ((g32 - r32).abs() <= r32.abs() * 2 ** -7 + 1e-5 * r32.abs().max()).all()
    rows = torch.tensor([0, 127, 128, M - 1])
    want = o8.mxfp8_gemm_ref(a[rows.to(dev)].cpu(), asc[rows.to(dev)].cpu(), b.cpu(), bsc.cpu())
    assert _rel_err(got[rows.to(dev)].float().cpu(), want) < (HW_SUM if out_dtype == "float32" else REL)


def test_mxfp8_stream_contract(dev):
    """What the streamed kernels cannot take is refused by name, and the automatic choice falls back."""
    import iree_turbine_amd as ita
    from oracle import inputs, mxfp8 as o8

    announce("mxfp8 streamed contract")
    names = ita._lib.variants("mxfp8_gemm")
    for (M, N, K) in [(256, 256, 512), (256, 256, 1280), (128, 256, 1024)]:  # K < 1024, K % 512 != 0, M % 256 != 0
        a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp8_inputs(M, N, K, seed=2)]
        for vn in ("stream_256x256x128_w2x2", "stream_256x256x128_w2x2_walk"):
            with pytest.raises(ValueError, match="stream_256x256x128"):
                torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, "bfloat16", names.index(vn))
        got = torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, "float32", -1)
        assert _rel_err(got.cpu(), o8.mxfp8_gemm_ref(a.cpu(), asc.cpu(), b.cpu(), bsc.cpu())) < HW_SUM
    # scale rows that are not 16-byte aligned: the streamed kernel loads scale groups 16 bytes at a time
    M, N, K = 256, 256, 1024
    a, asc, b, bsc = [t.to(dev) for t in inputs.mxfp8_inputs(M, N, K, seed=2)]
    pad = torch.zeros(M * (K // 32) + 4, dtype=torch.uint8, device=dev)
    asc_off = pad[4:].view(M, K // 32)
    asc_off.copy_(asc)
    with pytest.raises(ValueError, match="stream_256x256x128"):
        torch.ops.mi355.mxfp8_gemm(a, asc_off, b, bsc, "bfloat16", names.index("stream_256x256x128_w2x2"))
    got = torch.ops.mi355.mxfp8_gemm(a, asc_off, b, bsc, "float32", -1)
    assert _rel_err(got, torch.ops.mi355.mxfp8_gemm(a, asc, b, bsc, "float32", names.index("generic_32x128"))) < HW_SUM


def test_mxfp8_contract_errors(dev):
    import iree_turbine_amd  # noqa: F401

    a = torch.zeros(256, 48, dtype=torch.uint8, device=dev)
    s = torch.zeros(256, 1, dtype=torch.uint8, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp8_gemm(a, s, a, s, "bfloat16", -1)  # K = 48
    a = torch.zeros(256, 128, dtype=torch.uint8, device=dev)
    s = torch.zeros(256, 4, dtype=torch.uint8, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp8_gemm(a, s, a, s, "bfloat16", 0)  # tiled kernel needs K % 256 == 0
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp8_gemm(a, s, a, s, "float16", -1)
    a = torch.zeros(256, 256, dtype=torch.uint8, device=dev)
    s = torch.zeros(256, 8, dtype=torch.uint8, device=dev)
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp8_gemm(a, s, a, s, "bfloat16", 2)  # the staged kernel needs four slabs
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp8_gemm(a, s, a, s, "bfloat16", 3)  # no such variant


@pytest.mark.parametrize("shape", [(256, 512, 1024), (100, 70, 96), (1, 1, 32)])
def test_fp8_gemm_plain(dev, shape):
    """The GEMM without block scales: torch.float8_e4m3fn operands in, alpha applied to the fp32 sums; equal to
    the block-scaled kernel with every scale byte 127."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, mxfp8 as o8

    M, N, K = shape
    announce(f"fp8_gemm {shape}")
    a, _, b, _ = inputs.mxfp8_inputs(M, N, K, seed=9)
    alpha = 0.0625 * 3
    ref = o8.fp8_gemm_ref(a, b, alpha)
    got = torch.ops.mi355.fp8_gemm(a.to(dev).view(torch.float8_e4m3fn), b.to(dev).view(torch.float8_e4m3fn), alpha, "float32", -1)
    assert _rel_err(got.cpu(), ref) < HW_SUM
    ones_a = torch.full((M, K // 32), 127, dtype=torch.uint8, device=dev)
    ones_b = torch.full((N, K // 32), 127, dtype=torch.uint8, device=dev)
    scaled = torch.ops.mi355.mxfp8_gemm(a.to(dev), ones_a, b.to(dev), ones_b, "float32", -1)
    assert torch.equal(got, alpha * scaled)
    bf = torch.ops.mi355.fp8_gemm(a.to(dev), b.to(dev), alpha, "bfloat16", -1)
    assert torch.equal(bf, got.bfloat16())
    if M % 256 == 0:  # the tiled kernels, chosen explicitly: each pair takes the k blocks in the same order
        by_variant = [torch.ops.mi355.fp8_gemm(a.to(dev), b.to(dev), alpha, "float32", variant) for variant in range(5)]
        assert torch.equal(by_variant[0], by_variant[2])
        assert torch.equal(by_variant[3], by_variant[4])
        for variant in range(5):
            assert _rel_err(by_variant[variant].cpu(), ref) < HW_SUM, variant
        assert torch.equal(got, by_variant[4])  # the automatic choice here
        bf = torch.ops.mi355.fp8_gemm(a.to(dev), b.to(dev), alpha, "bfloat16", 3)
        assert torch.equal(bf, by_variant[3].bfloat16())
    # against torch's own decode of the same bytes
    lib = alpha * (a.view(torch.float8_e4m3fn).float() @ b.view(torch.float8_e4m3fn).float().t())
    assert _rel_err(got.cpu(), lib) < HW_SUM
