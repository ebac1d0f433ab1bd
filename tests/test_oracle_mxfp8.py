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
