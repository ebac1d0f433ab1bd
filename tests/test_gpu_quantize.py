"""GPU parity: MXFP4 quantisation through the C ABI, bit for bit against the oracle (codes and scale bytes)."""

import numpy as np
import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu


def _check(dev, x: torch.Tensor):
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp4 as om

    codes, scales = torch.ops.mi355.mxfp4_quantize(x.to(dev))
    rc, rs = om.mxfp4_quantize_ref(x)
    assert codes.dtype == torch.uint8 and tuple(codes.shape) == rc.shape and tuple(scales.shape) == rs.shape
    assert np.array_equal(scales.cpu().numpy(), rs)
    assert np.array_equal(codes.cpu().numpy(), rc)
    return codes, scales


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 32), (3, 96), (7, 544), (64, 4096), (33, 1056)])
def test_quantize_random(dev, dtype, shape):
    announce(f"mxfp4_quantize random {shape} {dtype}")
    g = torch.Generator().manual_seed(shape[0] * 1000 + shape[1])
    x = torch.randn(shape, generator=g) * torch.exp(torch.randn(shape[0], 1, generator=g) * 3)
    _check(dev, x.to(dtype))


def test_quantize_ties_saturation_and_specials(dev):
    announce("mxfp4_quantize special values")
    rows = []
    ties = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 5.0001, 0.2499, 6.0, -0.75, -0.0, 0.0, -5.0, 3.4999, 1.0]
    for e in (-20, -3, 0, 5, 12):
        rows.append([4.0 * 2.0 ** e] + [t * 2.0 ** e for t in ties] + [0.0] * 15)       # shared exponent e
    rows.append([7.99, -7.5, 6.1] + [0.0] * 29)                                          # top-binade saturation
    rows.append([0.0] * 31 + [-0.0])                                                     # all zero
    rows.append([1.0, float("nan")] + [2.0] * 30)
    rows.append([float("-inf")] + [1.0] * 31)
    rows.append([65504.0, -65504.0] + [1000.0] * 30)                                     # fp16 maximum
    rows.append([6.0e-8, 5.96e-8, -1.2e-7] + [0.0] * 29)                                 # fp16 subnormals
    x = torch.tensor(rows, dtype=torch.float32)
    for dt in (torch.float16, torch.float32, torch.bfloat16):
        _check(dev, x.to(dt))
    big = torch.tensor([[3.0e38, -1.0e38, 2.0 ** -140, 2.0 ** -149] + [0.0] * 28, [2.0 ** -140] + [0.0] * 31], dtype=torch.float32)
    _check(dev, big)                                                                     # exponent clamps at both ends
    _check(dev, big.to(torch.bfloat16))


def test_quantize_feeds_the_gemm(dev):
    """Quantise fp16 operands on the device, multiply with the block-scaled GEMM, compare with the fp32
    product of the dequantised operands (<= 1e-5) and with the product of the original operands (the
    format's own error, a few percent)."""
    import iree_turbine_amd  # noqa: F401

    announce("mxfp4_quantize -> mxfp4_gemm")
    g = torch.Generator().manual_seed(3)
    a = (torch.randn(512, 2048, generator=g)).half().to(dev)
    b = (torch.randn(768, 2048, generator=g)).half().to(dev)
    ac, asc = torch.ops.mi355.mxfp4_quantize(a)
    bc, bsc = torch.ops.mi355.mxfp4_quantize(b)
    c = torch.ops.mi355.mxfp4_gemm(ac, asc, bc, bsc, "float32", -1)
    da, db = torch.ops.mi355.mxfp4_dequant(ac, asc), torch.ops.mi355.mxfp4_dequant(bc, bsc)
    ref = da.double() @ db.double().t()
    assert ((c.double() - ref).norm() / ref.norm()).item() < 1e-5
    exact = a.double() @ b.double().t()
    assert ((c.double() - exact).norm() / exact.norm()).item() < 0.2
    # the dequantised tensors are fixed points of the quantiser
    ac2, asc2 = torch.ops.mi355.mxfp4_quantize(da)
    assert torch.equal(torch.ops.mi355.mxfp4_dequant(ac2, asc2), da)


def test_quantize_full_size_and_contract(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import mxfp4 as om

    announce("mxfp4_quantize 4096x8192")
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(4096, 8192, generator=g) * 0.1).half()
    codes, scales = torch.ops.mi355.mxfp4_quantize(x.to(dev))
    rows = torch.tensor([0, 1, 2047, 4095])
    rc, rs = om.mxfp4_quantize_ref(x[rows])
    assert np.array_equal(codes[rows.to(dev)].cpu().numpy(), rc) and np.array_equal(scales[rows.to(dev)].cpu().numpy(), rs)
    # every block's largest magnitude code is 4, 5, 6 or 7 (the maximum lands in the top binade [4, 8))
    mags = torch.maximum(codes & 7, (codes >> 4) & 7).view(4096, 256, 16).amax(dim=2)
    assert (mags >= 6).all()
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp4_quantize(torch.zeros(4, 48, dtype=torch.float16, device=dev))
    with pytest.raises(ValueError):
        torch.ops.mi355.mxfp4_quantize(torch.zeros(4, 64, dtype=torch.float64, device=dev))
