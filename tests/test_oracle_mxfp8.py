"""Pins of the MXFP8 oracle (CPU): the E4M3 decode against torch's own float8_e4m3fn and the format's spec
values, the block scaling against hand-computed cases, and the GEMM oracle against float64 and exact cases."""

import numpy as np
import torch

from oracle import inputs, mxfp8 as o8


def test_e4m3_table_vs_torch_library_and_spec_values():
    codes = torch.arange(256, dtype=torch.uint8)
    lib = codes.view(torch.float8_e4m3fn).float().numpy()
    ours = o8.E4M3_VALUES
    nan = np.isnan(lib)
    assert np.array_equal(nan, np.isnan(ours)) and set(np.nonzero(nan)[0]) == {0x7F, 0xFF}
    assert np.array_equal(lib[~nan].view(np.uint32), ours[~nan].view(np.uint32))  # bit-exact, signed zeros included
    # spec values: largest finite 448, smallest normal 2^-6, smallest subnormal 2^-9, no infinities
    assert ours[0x7E] == 448.0 and ours[0xFE] == -448.0
    assert ours[0x08] == 2.0 ** -6 and ours[0x01] == 2.0 ** -9
    assert np.isfinite(ours[~nan]).all()
    assert ours[0x38] == 1.0 and ours[0x40] == 2.0 and ours[0x3C] == 1.5


def test_block_scaling_hand_cases():
    K = 64
    codes = np.zeros((2, K), dtype=np.uint8)
    codes[0, :] = 0x38          # 1.0 everywhere
    codes[1, 0] = 0x7E          # 448 in block 0
    codes[1, 32] = 0xC0         # -2 in block 1
    scales = np.array([[127, 130], [120, 127 + 8]], dtype=np.uint8)
    out = o8.mxfp8_dequant_ref(codes, scales)
    assert (out[0, :32] == 1.0).all() and (out[0, 32:] == 8.0).all()
    assert out[1, 0] == 448.0 * 2.0 ** -7 and out[1, 32] == -2.0 * 256.0
    assert (out[1, 1:32] == 0).all()


def test_gemm_oracle_exact_and_vs_float64():
    # one-hot: a single non-zero product lands in the right cell with the right scale
    K = 128
    a = np.zeros((3, K), dtype=np.uint8); b = np.zeros((4, K), dtype=np.uint8)
    a[1, 70] = 0x3C   # 1.5, block 2
    b[2, 70] = 0xC8   # -4, block 2
    sa = np.full((3, 4), 127, dtype=np.uint8); sb = np.full((4, 4), 127, dtype=np.uint8)
    sa[1, 2] = 129; sb[2, 2] = 124
    c = o8.mxfp8_gemm_ref(torch.from_numpy(a), torch.from_numpy(sa), torch.from_numpy(b), torch.from_numpy(sb))
    want = torch.zeros(3, 4); want[1, 2] = 1.5 * 4 * -4.0 / 8
    assert torch.equal(c, want)
    # random: fp32 accumulation against float64
    A, As, B, Bs = inputs.mxfp8_inputs(48, 40, 512, seed=3)
    c32, c64 = o8.mxfp8_gemm_ref(A, As, B, Bs), o8.mxfp8_gemm_f64(A, As, B, Bs)
    assert ((c32.double() - c64).abs().max() / c64.abs().max()).item() < 1e-6
    # scaling law: raising every A scale by one doubles the result exactly
    c2 = o8.mxfp8_gemm_ref(A, As + 1, B, Bs)
    assert torch.equal(c2, 2 * c32)
    # inputs never hold a NaN code
    assert not (((A & 0x7F) == 0x7F).any() or ((B & 0x7F) == 0x7F).any())


def test_plain_fp8_gemm_oracle_vs_torch_decode():
    A, _, B, _ = inputs.mxfp8_inputs(20, 24, 96, seed=4)
    ref = o8.fp8_gemm_ref(A, B, 0.5)
    lib = 0.5 * (A.view(torch.float8_e4m3fn).float() @ B.view(torch.float8_e4m3fn).float().t())
    assert torch.equal(ref, lib)
    assert torch.equal(o8.fp8_gemm_ref(A.view(torch.float8_e4m3fn), B, 0.5), ref)


def test_quantize_oracle_rounding_vs_torch_library_and_spec_cases():
    """The nearest-code search against torch's own float -> float8_e4m3fn conversion on every midpoint, every
    representable value and random magnitudes up to the largest finite value; block exponents by hand."""
    from oracle import mxfp8 as o8

    g = torch.Generator().manual_seed(0)
    pos = o8.E4M3_VALUES[:127].astype(np.float64)
    mids = (pos[:-1] + pos[1:]) / 2
    y = np.concatenate([pos, mids, np.nextafter(mids.astype(np.float32), 0).astype(np.float64),
                        np.nextafter(mids.astype(np.float32), 1e9).astype(np.float64),
                        (torch.rand(50000, generator=g, dtype=torch.float64) * 448).numpy(),
                        (torch.rand(5000, generator=g, dtype=torch.float64) * 0.04).numpy()])
    lib = torch.from_numpy(y).float().to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(o8.e4m3_round(y), lib)
    assert o8.e4m3_round(np.array([449.0, 464.0, 1e6]))[...].tolist() == [0x7E, 0x7E, 0x7E]  # saturation at 448
    # ties go to the even code: 0.5 * 2^-9 -> 0, 1.5 * 2^-9 -> 2, 17 (between 16 and 18) -> 16 (code 0x58)
    assert o8.e4m3_round(np.array([2.0 ** -10, 3 * 2.0 ** -10, 17.0])).tolist() == [0, 2, 0x58]

    # block exponent: amax 1.0 -> shared -8 -> 1.0 becomes 256 = 0x78, scale byte 119
    x = torch.zeros(4, 32)
    x[0, 0], x[0, 1] = 1.0, -0.5
    x[1, :] = 0.0
    x[2, 3] = float("nan")
    x[2, 4] = -3.0
    x[3, 0], x[3, 1] = 7.9, 3.0  # 7.9 * 2^6 = 505.6 saturates to 448; 3 * 64 = 192 = 0x74
    codes, scales = o8.mxfp8_quantize_ref(x)
    assert scales[:, 0].tolist() == [119, 0, 255, 121]
    assert codes[0, :2].tolist() == [0x78, 0xF0] and not codes[1].any()
    assert codes[2, 4] == 0x80 and codes[2, 0] == 0
    assert codes[3, :2].tolist() == [0x7E, 0x74]
    # a representable tensor survives the round trip exactly
    g2 = torch.Generator().manual_seed(4)
    c0 = torch.randint(0, 256, (16, 64), generator=g2).to(torch.uint8)
    c0 = torch.where((c0 & 0x7F) == 0x7F, c0 - 1, c0)
    s0 = (127 + torch.randint(-20, 20, (16, 2), generator=g2)).to(torch.uint8)
    back = o8.mxfp8_dequant_ref(*o8.mxfp8_quantize_ref(torch.from_numpy(o8.mxfp8_dequant_ref(c0, s0))))
    assert np.array_equal(back, o8.mxfp8_dequant_ref(c0, s0))
