"""GPU parity: MXFP6 quantisation through the C ABI, bit for bit against the oracle (packed codes and scale bytes)."""

import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

FMTS = ["e2m3", "e3m2"]


def _check(dev, x: torch.Tensor, fmt: str):
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp6 as o6

    codes, scales = torch.ops.mi355.mxfp6_quantize(x.to(dev), fmt)
    rc, rs = o6.mxfp6_quantize_ref(x, fmt)
    assert codes.dtype == torch.uint8 and tuple(codes.shape) == rc.shape and tuple(scales.shape) == rs.shape
    assert np.array_equal(scales.cpu().numpy(), rs)
    got, want = o6.unpack_fp6(codes.cpu()), o6.unpack_fp6(rc)
    bad = np.argwhere(got != want)
    assert bad.size == 0, (fmt, bad[:5], got[tuple(bad[0])], want[tuple(bad[0])], x[tuple(bad[0])].item())
    assert np.array_equal(codes.cpu().numpy(), rc)
    return codes, scales


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 32), (3, 96), (7, 544), (64, 4096), (33, 1056)])
def test_quantize6_random(dev, dtype, shape, fmt):
    announce(f"mxfp6_quantize random {shape} {dtype} {fmt}")
    g = torch.Generator().manual_seed(shape[0] * 1000 + shape[1])
    x = torch.randn(shape, generator=g) * torch.exp(torch.randn(shape[0], 1, generator=g) * 3)
    _check(dev, x.to(dtype), fmt)


@pytest.mark.parametrize("fmt", FMTS)
def test_quantize6_every_fp16_value(dev, fmt):
    """Every fp16 bit pattern as an element of a block whose maximum fixes the shared exponent: all roundings of
    the hardware conversion (normal and subnormal codes, ties, saturation) against the nearest-value search."""
    announce(f"mxfp6_quantize all fp16 values {fmt}")
    vals = torch.arange(0, 65536, dtype=torch.int32).to(torch.uint16).view(torch.float16)
    finite = vals[torch.isfinite(vals.float())]
    n = (finite.numel() + 30) // 31 * 31
    finite = torch.cat([finite, torch.zeros(n - finite.numel(), dtype=torch.float16)])
    for top in (1.0, 300.0, 65504.0, 0.01, 7.9):
        x = torch.empty(n // 31, 32, dtype=torch.float16)
        x[:, 0] = top
        x[:, 1:] = finite.view(-1, 31)
        x[:, 1:] = torch.where(x[:, 1:].float().abs() > top, torch.zeros_like(x[:, 1:]), x[:, 1:])
        _check(dev, x, fmt)
        _check(dev, x.float(), fmt)


@pytest.mark.parametrize("fmt", FMTS)
def test_quantize6_specials(dev, fmt):
    announce(f"mxfp6_quantize special values {fmt}")
    rows = []
    ties = [0.0625, 0.1875, 1.0625, 1.1875, 7.5, 7.75, 3.875, -1.0625, -0.0, 0.0, 5.25, 5.75, 26.0, 30.0, -28.0, 0.03125]
    for e in (-20, -3, 0, 5, 12):
        rows.append([4.0 * 2.0 ** e] + [t * 2.0 ** (e - 2) for t in ties] + [0.0] * 15)
    rows.append([7.99, -7.5, 6.1] + [0.0] * 29)
    rows.append([0.0] * 31 + [-0.0])
    rows.append([1.0, float("nan")] + [-2.0] * 30)
    rows.append([float("-inf")] + [1.0] * 31)
    rows.append([65504.0, -65504.0] + [1000.0] * 30)
    rows.append([6.0e-8, 5.96e-8, -1.2e-7] + [0.0] * 29)
    x = torch.tensor(rows, dtype=torch.float32)
    for dt in (torch.float16, torch.float32, torch.bfloat16):
        _check(dev, x.to(dt), fmt)
    big = torch.tensor([[3.0e38, -1.0e38, 2.0 ** -140, 2.0 ** -149] + [0.0] * 28, [2.0 ** -140] + [0.0] * 31,
                        [2.0 ** -126, -(2.0 ** -127), 2.0 ** -128] + [2.0 ** -130] * 29], dtype=torch.float32)
    _check(dev, big, fmt)                                   # exponent clamps at both ends, denormal scales
    _check(dev, big.to(torch.bfloat16), fmt)


def test_quantize6_feeds_the_gemm(dev):
    """Quantise fp16 operands on the device, multiply with the block-scaled GEMM; the dequantised tensors are
    fixed points of the quantiser."""
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp6 as o6

    announce("mxfp6_quantize -> mxfp6_gemm")
    g = torch.Generator().manual_seed(3)
    a = (torch.randn(512, 2048, generator=g)).half().to(dev)
    b = (torch.randn(768, 2048, generator=g)).half().to(dev)
    for fmt, fmt_err in (("e2m3", 0.06), ("e3m2", 0.1)):
        ac, asc = torch.ops.mi355.mxfp6_quantize(a, fmt)
        bc, bsc = torch.ops.mi355.mxfp6_quantize(b, fmt)
        c = torch.ops.mi355.mxfp6_gemm(ac, asc, bc, bsc, fmt, "float32", -1)
        da = torch.from_numpy(o6.mxfp6_dequant_ref(ac, asc, fmt)).double()
        db = torch.from_numpy(o6.mxfp6_dequant_ref(bc, bsc, fmt)).double()
        ref = da @ db.t()
        assert ((c.cpu().double() - ref).norm() / ref.norm()).item() < 5e-4
        exact = a.cpu().double() @ b.cpu().double().t()
        assert ((c.cpu().double() - exact).norm() / exact.norm()).item() < fmt_err
        ac2, asc2 = torch.ops.mi355.mxfp6_quantize(da.float().to(dev), fmt)
        assert np.array_equal(o6.mxfp6_dequant_ref(ac2, asc2, fmt), da.float().numpy())


def test_quantize6_full_size_and_contract(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp6 as o6

    announce("mxfp6_quantize 4096x8192")
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(4096, 8192, generator=g) * 0.1).half()
    codes, scales = torch.ops.mi355.mxfp6_quantize(x.to(dev), "e2m3")
    rows = torch.tensor([0, 1, 2047, 4095])
    rc, rs = o6.mxfp6_quantize_ref(x[rows], "e2m3")
    assert np.array_equal(codes[rows.to(dev)].cpu().numpy(), rc) and np.array_equal(scales[rows.to(dev)].cpu().numpy(), rs)
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp6_quantize(torch.zeros(4, 48, dtype=torch.float16, device=dev), "e2m3")
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp6_quantize(torch.zeros(4, 64, dtype=torch.float64, device=dev), "e2m3")
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp6_quantize(torch.zeros(4, 64, dtype=torch.float16, device=dev), "e4m3")
