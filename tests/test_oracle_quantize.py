"""Pins for the MXFP4 quantisation oracle: brute-force nearest rounding with ties to the even code, the
shared-exponent formula against math.frexp, exact round trips, idempotence and the error bound of the
format.  The reference holds no quantiser; the definition is OCP Microscaling Formats v1.0."""

import math

import numpy as np
import pytest
import torch

from oracle import mxfp4 as om


def _one_block(vals):
    x = np.zeros((1, 32))
    x[0, :len(vals)] = vals
    codes, scales = om.mxfp4_quantize_ref(x)
    return om.unpack_codes(codes)[0, :len(vals)], int(scales[0, 0])


def test_rounding_matches_brute_force_nearest_even():
    # amax = 4 pins the shared exponent at 0, so the other elements are rounded as they are
    ys = np.concatenate([np.linspace(0, 6.5, 2601), np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])])
    for chunk in np.array_split(ys, 120):
        codes, scale = _one_block([4.0] + list(chunk))
        assert scale == 127
        for y, c in zip(chunk, codes[1:]):
            assert c == om.e2m1_round_brute_force(float(y)), y
    # the ties, spelled out: .25->0, .75->1, 1.25->1, 1.75->2, 2.5->2, 3.5->4, 5->4 (even codes 0,2,2,4,4,6,6)
    codes, _ = _one_block([4.0, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.75, -0.0])
    assert list(codes[1:]) == [0, 2, 2, 4, 4, 6, 6, 8 | 2, 8]


@pytest.mark.parametrize("amax", [1e-30, 3e-5, 0.4999, 0.5, 1.0, 1.9999, 5.99, 6.0, 7.9, 8.0, 1000.0, 65504.0, 3.0e38])
def test_shared_exponent_formula(amax):
    _, scale = _one_block([amax, -amax / 3])
    assert scale == min(max(math.frexp(amax)[1] - 1 - 2, -127), 127) + 127
    assert math.ldexp(8.0, scale - 127) > amax or scale == 254  # amax / scale < 8


def test_special_blocks():
    assert _one_block([0.0, -0.0])[1] == 0                                   # all zero: smallest scale
    assert list(_one_block([0.0, -0.0])[0]) == [0, 8]
    assert _one_block([1.0, float("nan")])[1] == 255
    codes, scale = _one_block([float("-inf"), 2.0, -3.0])                   # NaN scale; magnitudes zero, signs kept
    assert scale == 255 and list(codes) == [8, 0, 8]
    codes, scale = _one_block([7.99, -7.5, 6.1])                            # saturation inside the top binade
    assert scale == 127 and list(codes) == [7, 15, 7]
    tiny = 2.0 ** -140                                                       # exponent clamps at -127
    codes, scale = _one_block([tiny])
    assert scale == 0 and codes[0] == 0


def test_round_trip_idempotence_and_error_bound():
    g = np.random.default_rng(0)
    # exact round trip: grid values times a power of two per block, with the block maximum in [4, 6]
    codes = g.integers(0, 16, size=(64, 256)).astype(np.uint8)
    codes[:, ::32] = 7
    scales = g.integers(100, 150, size=(64, 8)).astype(np.uint8)
    x = om.mxfp4_dequant_ref(om.pack_codes(codes), scales)
    c2, s2 = om.mxfp4_quantize_ref(x)
    assert np.array_equal(s2, scales)
    assert np.array_equal(om.mxfp4_dequant_ref(c2, s2), x)
    # random data: idempotent, and within half a grid step (a full step only in the saturated top binade)
    x = (g.standard_normal((128, 512)) * np.exp(g.standard_normal((128, 1)) * 3)).astype(np.float32)
    c, s = om.mxfp4_quantize_ref(x)
    dq = om.mxfp4_dequant_ref(c, s)
    c3, s3 = om.mxfp4_quantize_ref(dq)
    assert np.array_equal(c3, c)
    assert (s3 <= s).all()  # a block whose maximum rounded down may need a smaller exponent the second time
    assert np.array_equal(om.mxfp4_dequant_ref(c3, s3), dq)
    scale = np.repeat(om.e8m0_decode(s), 32, axis=1).astype(np.float64)
    y = np.abs(x) / scale
    step = np.where(y < 2, 0.5, np.where(y < 4, 1.0, 2.0))
    assert (np.abs(dq.astype(np.float64) - x) <= np.where(y <= 6, step / 2, 2.0) * scale * (1 + 1e-12)).all()
    assert (y < 8).all()


def test_torch_dtypes_accepted():
    x = torch.randn(4, 64)
    for dt in (torch.float16, torch.bfloat16, torch.float32):
        c, s = om.mxfp4_quantize_ref(x.to(dt))
        c2, s2 = om.mxfp4_quantize_ref(x.to(dt).double())
        assert np.array_equal(c, c2) and np.array_equal(s, s2)
