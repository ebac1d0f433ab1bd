"""Pins the paged-decode and MXFP4 oracles (closed forms, library decode of the scale format, brute
force, the C restatement, invariants)."""

import ctypes
import math
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import attention as oa, inputs, mxfp4 as om, paged_decode as op


def test_paged_decode_equals_dense_attention_on_contiguous_cache():
    S, Hq, Hkv, D, page = 3, 8, 2, 16, 16
    g = torch.Generator().manual_seed(1)
    lens = torch.tensor([16, 40, 7], dtype=torch.int32)
    n_pg = (lens + page - 1) // page
    P = int(n_pg.sum())
    kc = torch.randn(P, page, Hkv, D, generator=g).half()
    vc = torch.randn(P, page, Hkv, D, generator=g).half()
    q = torch.randn(S, Hq, D, generator=g).half()
    bt = torch.full((S, int(n_pg.max())), -1, dtype=torch.int32)
    off = 0
    for s in range(S):
        bt[s, :n_pg[s]] = torch.arange(off, off + int(n_pg[s]), dtype=torch.int32)
        off += int(n_pg[s])
    out = op.paged_decode_ref(q, kc, vc, bt, lens)
    off = 0
    for s in range(S):
        ln = int(lens[s])
        ks = kc[off:off + int(n_pg[s])].reshape(-1, Hkv, D)[:ln]
        vs = vc[off:off + int(n_pg[s])].reshape(-1, Hkv, D)[:ln]
        off += int(n_pg[s])
        for h in range(Hq):
            kv = h // (Hq // Hkv)  # the GQA rule: q head h reads kv head h // n_rep
            ref = oa.sdpa_ref(q[s, h][None], ks[:, kv], vs[:, kv])[0]
            torch.testing.assert_close(out[s, h], ref, rtol=1e-5, atol=1e-6)


def test_paged_decode_invariances_and_poison():
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=4, num_q_heads=4, num_kv_heads=2, D=16, min_len=1, max_len=90, seed=3)
    base = op.paged_decode_ref(q, kc, vc, bt, sl)
    P = kc.shape[0]
    perm = torch.randperm(P, generator=torch.Generator().manual_seed(2))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(P)
    bt2 = torch.where(bt >= 0, inv[bt.clamp(min=0).long()].int(), bt)
    assert torch.equal(op.paged_decode_ref(q, kc[perm], vc[perm], bt2, sl), base)  # physical placement is irrelevant
    # tokens past the length never matter
    kp, vp = kc.clone(), vc.clone()
    for s in range(4):
        ln = int(sl[s])
        last = int(bt[s, (ln - 1) // 16])
        if ln % 16:
            kp[last, ln % 16:] = float("nan")
            vp[last, ln % 16:] = float("nan")
    assert torch.equal(op.paged_decode_ref(q, kp, vp, bt, sl), base)
    assert inputs.paged_decode_inputs(num_seqs=2, min_len=5, max_len=5, D=16)[3].shape[1] == 1
    # repeat_kv ordering
    x = torch.arange(2 * 3 * 1).float().view(2, 3, 1)
    assert op.repeat_kv(x, 2)[:, :, 0].tolist() == [[0, 0, 1, 1, 2, 2], [3, 3, 4, 4, 5, 5]]


def test_e2m1_table_closed_form_and_spec_values():
    assert [om.e2m1_closed_form(c) for c in range(16)] == list(om.E2M1_VALUES)
    # OCP MX v1.0 table 5: magnitudes 0, 0.5, 1, 1.5, 2, 3, 4, 6; code 0x8 is negative zero
    assert om.E2M1_VALUES[:8] == (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
    assert math.copysign(1.0, om.E2M1_VALUES[8]) == -1.0 and om.E2M1_VALUES[8] == 0.0
    assert all(om.E2M1_VALUES[c + 8] == -om.E2M1_VALUES[c] for c in range(8))


def test_e8m0_decode_vs_torch_library():
    b = np.arange(256, dtype=np.uint8)
    ours = om.e8m0_decode(b)
    lib = torch.from_numpy(b.copy()).view(torch.float8_e8m0fnu).to(torch.float32).numpy()
    assert np.array_equal(ours[:255].view(np.uint32), lib[:255].view(np.uint32))
    assert np.isnan(ours[255]) and np.isnan(lib[255])
    assert ours[127] == 1.0 and ours[119] == 2.0**-8 and ours[135] == 256.0 and ours[0] == 2.0**-127


def test_dequant_exhaustive_products_exact_in_bf16():
    packed = om.pack_codes(np.tile(np.arange(16, dtype=np.uint8), 2)[None, :].repeat(17, 0))
    scales = (119 + np.arange(17, dtype=np.uint8))[:, None]
    dq = om.mxfp4_dequant_ref(packed, scales)
    for r in range(17):
        for k in range(32):
            assert dq[r, k] == om.E2M1_VALUES[k % 16] * 2.0 ** (int(scales[r, 0]) - 127)
    t = torch.from_numpy(dq)
    assert torch.equal(t.bfloat16().float(), t)  # every value is bf16-representable


def test_pack_unpack_nibble_order():
    codes = np.array([[1, 2, 3, 4]], dtype=np.uint8)
    packed = om.pack_codes(codes)
    assert packed.tolist() == [[0x21, 0x43]]  # element 0 in the low nibble
    assert np.array_equal(om.unpack_codes(packed), codes)


def _c_oracle():
    so = Path(__file__).resolve().parent.parent / "oracle" / "_build" / "libmxfp4_ref.so"
    if not so.exists():
        from oracle.build_oracle import build_oracle
        build_oracle()
    lib = ctypes.CDLL(str(so))
    return lib


def test_python_oracle_vs_c_restatement():
    lib = _c_oracle()
    a, asc, b, bsc = inputs.mxfp4_inputs(9, 7, 96, seed=5)
    out = np.empty((9, 96), dtype=np.float32)
    lib.mxfp4_dequant_c(a.numpy().ctypes.data_as(ctypes.c_void_p), asc.numpy().ctypes.data_as(ctypes.c_void_p),
                        out.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(9), ctypes.c_int64(96))
    assert np.array_equal(out.view(np.uint32), om.mxfp4_dequant_ref(a, asc).view(np.uint32))
    c = np.empty((9, 7), dtype=np.float32)
    lib.mxfp4_gemm_c(*(t.numpy().ctypes.data_as(ctypes.c_void_p) for t in (a, asc, b, bsc)), c.ctypes.data_as(ctypes.c_void_p),
                     ctypes.c_int64(9), ctypes.c_int64(7), ctypes.c_int64(96))
    np.testing.assert_allclose(c, om.mxfp4_gemm_f64(a, asc, b, bsc).numpy(), rtol=1e-6, atol=0)
    np.testing.assert_allclose(om.mxfp4_gemm_ref(a, asc, b, bsc).numpy(), c, rtol=1e-5, atol=1e-4)


def test_mxfp4_gemm_exact_cases_and_scaling_law():
    g = torch.Generator().manual_seed(3)
    pick = np.array([0, 2, 4, 6], dtype=np.uint8)
    ca = pick[torch.randint(0, 4, (8, 64), generator=g).numpy()]
    cb = pick[torch.randint(0, 4, (6, 64), generator=g).numpy()]
    a, b = om.pack_codes(ca), om.pack_codes(cb)
    one_a, one_b = np.full((8, 2), 127, np.uint8), np.full((6, 2), 127, np.uint8)
    vals = np.array([0, 1, 2, 4])
    exp = vals[ca // 2].astype(np.int64) @ vals[cb // 2].astype(np.int64).T
    assert np.array_equal(om.mxfp4_gemm_ref(a, one_a, b, one_b).numpy(), exp.astype(np.float32))
    assert np.array_equal(om.mxfp4_gemm_ref(a, one_a + 1, b, one_b).numpy(), 2 * exp.astype(np.float32))
    # a scale byte covers exactly 32 consecutive k
    sc = one_a.copy()
    sc[:, 1] = 128
    exp2 = vals[ca // 2][:, :32] @ vals[cb // 2][:, :32].T + 2 * (vals[ca // 2][:, 32:] @ vals[cb // 2][:, 32:].T)
    assert np.array_equal(om.mxfp4_gemm_ref(a, sc, b, one_b).numpy(), exp2.astype(np.float32))


def test_window_and_append_oracles():
    """Sliding window = dense attention over the last W tokens; append = slice assignment of a dense cache."""
    from oracle import inputs, paged_decode as op

    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=5, num_q_heads=8, num_kv_heads=2, min_len=3, max_len=90, seed=4)
    W = 20
    out = op.paged_decode_ref(q, kc, vc, bt, sl, window=W)
    assert torch.equal(op.paged_decode_ref(q, kc, vc, bt, sl, window=0), op.paged_decode_ref(q, kc, vc, bt, sl))
    for s in range(5):
        ln = int(sl[s])
        k = op.gather_kv(kc.float(), bt[s], ln)[max(0, ln - W):]            # [w, Hkv, D]
        v = op.gather_kv(vc.float(), bt[s], ln)[max(0, ln - W):]
        for h in range(8):
            p = torch.softmax((k[:, h // 4] @ q[s, h].float()) / 128 ** 0.5, dim=0)
            torch.testing.assert_close(out[s, h], p @ v[:, h // 4], rtol=1e-5, atol=1e-6)
    # append: a dense [S, max_len] cache gathered back through the table equals slice assignment
    S, n_new = 5, 7
    g = torch.Generator().manual_seed(1)
    start = torch.tensor([0, 3, 16, 25, int(sl[4]) - n_new], dtype=torch.int32)
    kn = torch.randn(S, n_new, 2, 128, generator=g).half()
    vn = torch.randn(S, n_new, 2, 128, generator=g).half()
    need = (start + n_new + 15) // 16
    bt2 = bt.clone()
    free = [p for p in range(kc.shape[0]) if p not in set(bt[bt >= 0].tolist())]
    assert not free  # every page is owned; give short sequences room by re-using their own table only
    ok = [s for s in range(S) if int(need[s]) <= int((sl[s] + 15) // 16)]
    k2, v2 = op.kv_cache_append_ref(kn, vn, kc, vc, bt2, start)
    for s in ok:
        ln = int(start[s]) + n_new
        dense = op.gather_kv(kc, bt[s], ln).clone()
        dense[int(start[s]):ln] = kn[s]
        assert torch.equal(op.gather_kv(k2, bt[s], ln), dense)
    assert len(ok) >= 2
    # a position beyond the table is skipped, not written elsewhere
    far = torch.full((S,), 16 * bt.shape[1], dtype=torch.int32)
    k3, v3 = op.kv_cache_append_ref(kn, vn, kc, vc, bt, far)
    assert torch.equal(k3, kc) and torch.equal(v3, vc)


def test_paged_prefill_oracle_reduces_to_known_cases():
    """One new token = the decode oracle; a chunk that is the whole sequence = causal SDPA over the gathered
    dense tensors; a chunk after a prefix = the last rows of causal SDPA over the whole sequence; a chunk longer
    than the sequence leaves its first queries (nothing visible) at zero."""
    from oracle import attention as oa, inputs, paged_decode as op

    q1, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=4, num_q_heads=8, num_kv_heads=2, min_len=5, max_len=70, seed=9)
    torch.testing.assert_close(op.paged_prefill_ref(q1[:, None], kc, vc, bt, sl)[:, 0], op.paged_decode_ref(q1, kc, vc, bt, sl),
                               rtol=1e-5, atol=1e-6)
    g = torch.Generator().manual_seed(2)
    T = 12
    q = torch.randn(4, T, 8, 128, generator=g).half()
    out = op.paged_prefill_ref(q, kc, vc, bt, sl)
    for s in range(4):
        ln = int(sl[s])
        k = op.repeat_kv(op.gather_kv(kc, bt[s], ln), 4).transpose(0, 1)[None]  # [1, Hq, ln, D]
        v = op.repeat_kv(op.gather_kv(vc, bt[s], ln), 4).transpose(0, 1)[None]
        if ln >= T:
            # queries for all ln positions, of which the chunk is the last T: plain square causal attention
            q_all = torch.zeros(1, 8, ln, 128, dtype=torch.float16)
            q_all[0, :, ln - T:] = q[s].transpose(0, 1)
            ref = oa.sdpa_ref(q_all, k, v, is_causal=True)[0, :, ln - T:].transpose(0, 1)
            torch.testing.assert_close(out[s], ref, rtol=1e-5, atol=1e-6)
        else:
            assert torch.equal(out[s, :T - ln], torch.zeros(T - ln, 8, 128))
            ref = oa.sdpa_ref(q[s, T - ln:].transpose(0, 1)[None], k, v, is_causal=True)[0].transpose(0, 1)
            torch.testing.assert_close(out[s, T - ln:], ref, rtol=1e-5, atol=1e-6)
    assert (sl < T).any() and (sl >= T).any()
