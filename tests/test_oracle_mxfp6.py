"""CPU: the MXFP6 oracle against the published format (OCP Microscaling Formats v1.0) and hand-worked cases."""

import numpy as np
import torch


def test_fp6_tables_against_spec_values():
    from oracle import mxfp6 as o6

    e2m3, e3m2 = o6.FP6_VALUES["e2m3"], o6.FP6_VALUES["e3m2"]
    # E2M3: subnormals k/8 for k = 0..7, then 1..1.875, 2..3.75, 4..7.5
    assert e2m3[:8].tolist() == [k / 8 for k in range(8)]
    assert e2m3[8:16].tolist() == [1 + k / 8 for k in range(8)]
    assert e2m3[16] == 2.0 and e2m3[24] == 4.0 and e2m3[31] == 7.5 and e2m3[63] == -7.5
    # E3M2: subnormals k/16, smallest normal 0.25, largest 28
    assert e3m2[:4].tolist() == [0.0, 0.0625, 0.125, 0.1875]
    assert e3m2[4] == 0.25 and e3m2[12] == 1.0 and e3m2[13] == 1.25 and e3m2[31] == 28.0 and e3m2[32 + 31] == -28.0
    for t in (e2m3, e3m2):
        assert np.all(np.diff(t[:32]) > 0)            # positive codes ascend
        assert np.array_equal(t[32:], -t[:32])        # bit 5 is the sign (code 32 is -0)
        assert np.all(np.isfinite(t))                 # no NaN or infinity codes


def test_fp6_packing_layout():
    """Element k at bits [6k, 6k+6) of the row: hand-packed bytes, and pack/unpack written two different ways."""
    from oracle import mxfp6 as o6

    # codes 1, 2, 3, 4 -> bits 000001 000010 000011 000100 (element 0 lowest) = 0x1 | 0x2<<6 | 0x3<<12 | 0x4<<18
    word = 1 | (2 << 6) | (3 << 12) | (4 << 18)
    want = [word & 255, (word >> 8) & 255, (word >> 16) & 255]
    assert o6.pack_fp6(np.array([[1, 2, 3, 4]])).tolist() == [want] == [[0x81, 0x30, 0x10]]
    one = np.zeros((1, 32), dtype=np.uint8)
    one[0, 5] = 63                                    # bits 30..35: byte 3 bits 6,7 and byte 4 bits 0..3
    p = o6.pack_fp6(one)
    assert p[0, 3] == 0xC0 and p[0, 4] == 0x0F and p.sum() == 0xC0 + 0x0F and p.shape == (1, 24)
    g = torch.Generator().manual_seed(1)
    codes = torch.randint(0, 64, (5, 96), generator=g).numpy().astype(np.uint8)
    assert np.array_equal(o6.unpack_fp6(o6.pack_fp6(codes)), codes)


def test_mxfp6_dequant_and_gemm_hand_cases():
    from oracle import inputs, mxfp6 as o6

    codes = np.zeros((2, 32), dtype=np.uint8)
    codes[0, 0], codes[0, 31], codes[1, 3] = 8, 63, 12   # e2m3: 1.0, -7.5, 1.5 ; e3m2: 0.5, -28, 1.0
    scales = np.array([[128], [125]], dtype=np.uint8)    # x2, x1/4
    dq = o6.mxfp6_dequant_ref(o6.pack_fp6(codes), scales, "e2m3")
    assert dq[0, 0] == 2.0 and dq[0, 31] == -15.0 and dq[1, 3] == 0.375 and np.count_nonzero(dq) == 3
    dq = o6.mxfp6_dequant_ref(o6.pack_fp6(codes), scales, "e3m2")
    assert dq[0, 0] == 1.0 and dq[0, 31] == -56.0 and dq[1, 3] == 0.25
    # small integers with unit scales: the fp32 product is exact and equals the float64 one
    g = torch.Generator().manual_seed(2)
    ints = torch.tensor([0, 8, 16, 24, 40, 48])[torch.randint(0, 6, (16, 64), generator=g)]  # 0, 1, 2, 4, -1, -2
    a = o6.pack_fp6(ints)
    s = np.full((16, 2), 127, dtype=np.uint8)
    c = o6.mxfp6_gemm_ref(a, s, a, s, "e2m3")
    assert torch.equal(c.double(), o6.mxfp6_gemm_f64(a, s, a, s, "e2m3")) and torch.equal(c, c.round())
    # +1 on every A scale byte doubles the result exactly
    a_, as_, b_, bs_ = inputs.mxfp6_inputs(8, 12, 128, seed=3)
    for fmt in ("e2m3", "e3m2"):
        c1 = o6.mxfp6_gemm_f64(a_, as_, b_, bs_, fmt)
        c2 = o6.mxfp6_gemm_f64(a_, as_ + 1, b_, bs_, fmt)
        assert torch.equal(c2, 2 * c1)


def test_mxfp6_quantize_oracle_hand_cases():
    from oracle import mxfp6 as o6

    # rounding: ties to the even code, saturation, subnormal steps (E2M3 step 1/8 below 1, E3M2 step 1/16 below 1/4)
    assert o6.fp6_round(np.array([0.0, 0.0625, 0.1875, 1.0625, 1.1875, 7.5, 7.75, 100.0, 3.875]), "e2m3").tolist() == [0, 0, 2, 8, 10, 31, 31, 31, 24]
    assert o6.fp6_round(np.array([0.03125, 0.09375, 0.25, 1.125, 1.375, 28.0, 30.0, 26.0]), "e3m2").tolist() == [0, 2, 4, 12, 14, 31, 31, 30]
    x = torch.zeros(4, 32)
    x[0, 0], x[0, 1] = 1.0, -0.5       # amax 1 -> E2M3 shared -2: 1.0 -> 4.0 (code 24), -0.5 -> -2.0 (code 32 + 16)
    x[2, 3], x[2, 4] = float("inf"), -3.0
    x[3, 0], x[3, 1] = 7.9, 3.0        # E2M3: shared 0 -> 7.9 saturates to 7.5 (31), 3.0 (code 20)
    packed, scales = o6.mxfp6_quantize_ref(x, "e2m3")
    codes = o6.unpack_fp6(packed)
    assert scales[:, 0].tolist() == [125, 0, 255, 127]
    assert codes[0, :2].tolist() == [24, 48] and not codes[1].any()
    assert codes[2, 4] == 32 and codes[2, 3] == 0
    assert codes[3, :2].tolist() == [31, 20]
    packed, scales = o6.mxfp6_quantize_ref(x, "e3m2")  # emax 4: amax 1 -> shared -4: 1.0 -> 16 (code 28)
    assert scales[:, 0].tolist() == [123, 0, 255, 125] and o6.unpack_fp6(packed)[0, 0] == 28
    # representable tensors survive the round trip exactly
    g = torch.Generator().manual_seed(4)
    for fmt in ("e2m3", "e3m2"):
        c0 = o6.pack_fp6(torch.randint(0, 64, (16, 64), generator=g))
        s0 = (127 + torch.randint(-20, 20, (16, 2), generator=g)).to(torch.uint8)
        dq = o6.mxfp6_dequant_ref(c0, s0, fmt)
        assert np.array_equal(o6.mxfp6_dequant_ref(*o6.mxfp6_quantize_ref(torch.from_numpy(dq), fmt), fmt), dq)
