"""GPU parity: MXFP8 quantisation through the C ABI, bit for bit against the oracle (codes and scale bytes)."""

import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu


def _check(dev, x: torch.Tensor):
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp8 as o8

    codes, scales = torch.ops.mi355.mxfp8_quantize(x.to(dev))
    rc, rs = o8.mxfp8_quantize_ref(x)
    assert codes.dtype == torch.uint8 and tuple(codes.shape) == rc.shape and tuple(scales.shape) == rs.shape
    assert np.array_equal(scales.cpu().numpy(), rs)
    got = codes.cpu().numpy()
    bad = np.argwhere(got != rc)
    assert bad.size == 0, (bad[:5], got[tuple(bad[0])], rc[tuple(bad[0])], x[tuple(bad[0])].item())
    return codes, scales


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 32), (3, 96), (7, 544), (64, 4096), (33, 1056)])
def test_quantize8_random(dev, dtype, shape):
    announce(f"mxfp8_quantize random {shape} {dtype}")
    g = torch.Generator().manual_seed(shape[0] * 1000 + shape[1])
    x = torch.randn(shape, generator=g) * torch.exp(torch.randn(shape[0], 1, generator=g) * 3)
    _check(dev, x.to(dtype))


def test_quantize8_every_fp16_value(dev):
    """Every fp16 bit pattern as an element of a block whose maximum fixes the shared exponent at several
    values: all roundings of the hardware conversion (normal and subnormal codes, ties, saturation) against
    the nearest-code search."""
    announce("mxfp8_quantize all fp16 values")
    vals = torch.arange(0, 65536, dtype=torch.int32).to(torch.uint16).view(torch.float16)
    finite = vals[torch.isfinite(vals.float())]
    n = (finite.numel() + 30) // 31 * 31
    finite = torch.cat([finite, torch.zeros(n - finite.numel(), dtype=torch.float16)])
    for top in (1.0, 300.0, 65504.0, 0.01, 7.9):
        x = torch.empty(n // 31, 32, dtype=torch.float16)
        x[:, 0] = top
        x[:, 1:] = finite.view(-1, 31)
        # elements above the block's declared maximum would move the exponent: clamp them to it
        x[:, 1:] = torch.where(x[:, 1:].float().abs() > top, torch.zeros_like(x[:, 1:]), x[:, 1:])
        _check(dev, x)


def test_quantize8_ties_saturation_and_specials(dev):
    announce("mxfp8_quantize special values")
    rows = []
    ties = [17.0, 18.0, 19.0, 2.0 ** -10, 3 * 2.0 ** -10, 447.0, 464.0, 480.0, -17.0, -0.0, 0.0, 1.0625, 1.1875, 250.0, 0.0009765625, -448.0]
    for e in (-20, -3, 0, 5, 12):
        rows.append([256.0 * 2.0 ** e] + [t * 2.0 ** e for t in ties] + [0.0] * 15)   # shared exponent e
    rows.append([7.99, -7.5, 6.1] + [0.0] * 29)                                        # top of the binade saturates
    rows.append([0.0] * 31 + [-0.0])
    rows.append([1.0, float("nan")] + [-2.0] * 30)
    rows.append([float("-inf")] + [1.0] * 31)
    rows.append([65504.0, -65504.0] + [1000.0] * 30)
    rows.append([6.0e-8, 5.96e-8, -1.2e-7] + [0.0] * 29)
    x = torch.tensor(rows, dtype=torch.float32)
    for dt in (torch.float16, torch.float32, torch.bfloat16):
        _check(dev, x.to(dt))
    big = torch.tensor([[3.0e38, -1.0e38, 2.0 ** -140, 2.0 ** -149] + [0.0] * 28, [2.0 ** -140] + [0.0] * 31], dtype=torch.float32)
    _check(dev, big)
    _check(dev, big.to(torch.bfloat16))


def test_quantize8_feeds_the_gemm(dev):
    """Quantise fp16 operands on the device, multiply with the block-scaled GEMM: close to the fp32 product of
    the dequantised operands (the unit's own summation error) and to the product of the original operands
    (the format's error, a few percent); the codes view as torch.float8_e4m3fn."""
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp8 as o8

    announce("mxfp8_quantize -> mxfp8_gemm")
    g = torch.Generator().manual_seed(3)
    a = (torch.randn(512, 2048, generator=g)).half().to(dev)
    b = (torch.randn(768, 2048, generator=g)).half().to(dev)
    ac, asc = torch.ops.mi355.mxfp8_quantize(a)
    bc, bsc = torch.ops.mi355.mxfp8_quantize(b)
    c = torch.ops.mi355.mxfp8_gemm(ac, asc, bc, bsc, "float32", -1)
    da = torch.from_numpy(o8.mxfp8_dequant_ref(ac, asc)).double()
    db = torch.from_numpy(o8.mxfp8_dequant_ref(bc, bsc)).double()
    ref = da @ db.t()
    assert ((c.cpu().double() - ref).norm() / ref.norm()).item() < 5e-4
    exact = a.cpu().double() @ b.cpu().double().t()
    assert ((c.cpu().double() - exact).norm() / exact.norm()).item() < 0.05
    # torch's decode of the same bytes, times the block scales, is the dequantised tensor
    lib = ac.view(torch.float8_e4m3fn).float().cpu() * torch.from_numpy(
        np.repeat(o8.e8m0_decode(asc.cpu().numpy()), 32, axis=1))
    assert torch.equal(lib.double(), da)
    # the dequantised tensors are fixed points of the quantiser
    ac2, asc2 = torch.ops.mi355.mxfp8_quantize(da.float().to(dev))
    assert np.array_equal(o8.mxfp8_dequant_ref(ac2, asc2), da.float().numpy())


def test_quantize8_full_size_and_contract(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp8 as o8

    announce("mxfp8_quantize 4096x8192")
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(4096, 8192, generator=g) * 0.1).half()
    codes, scales = torch.ops.mi355.mxfp8_quantize(x.to(dev))
    rows = torch.tensor([0, 1, 2047, 4095])
    rc, rs = o8.mxfp8_quantize_ref(x[rows])
    assert np.array_equal(codes[rows.to(dev)].cpu().numpy(), rc) and np.array_equal(scales[rows.to(dev)].cpu().numpy(), rs)
    # every block's largest magnitude lands in the top binade [256, 512), clamped at 448: exponent field 15
    top = (codes & 0x7F).view(4096, 256, 32).amax(dim=2)
    assert (top >= 0x78).all() and (top <= 0x7E).all()
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp8_quantize(torch.zeros(4, 48, dtype=torch.float16, device=dev))
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp8_quantize(torch.zeros(4, 64, dtype=torch.float64, device=dev))
