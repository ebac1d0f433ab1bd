"""GPU: the decode entry point that allocates nothing (split-K partials in the library's own device array) against
the entry point with caller-owned scratch, through the C ABI: bit-identical on two calls in a row, the second on
a smaller batch (which reuses the front of the array the first call filled), and over-large sizes rejected."""

import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu


def _both(dev, q, kc, vc, bt, sl, splits):
    from iree_turbine_amd import _lib

    lib = _lib.load()
    S, Hq, D = q.shape
    P, page, Hkv, _ = kc.shape
    q, kc, vc, bt, sl = (t.to(dev).contiguous() for t in (q, kc, vc, bt, sl))
    want = torch.full((S, Hq, D), 7.0, dtype=torch.float16, device=dev)
    got = torch.full((S, Hq, D), -7.0, dtype=torch.float16, device=dev)
    pacc = torch.empty((S, Hq, splits, D), dtype=torch.float32, device=dev)
    pml = torch.empty((S, Hq, splits, 2), dtype=torch.float32, device=dev)
    stream = _lib.current_stream_ptr(dev)
    sizes = (S, Hq, Hkv, D, page, bt.shape[1], P, splits)
    rc = lib.mi355_paged_decode_attn(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(), sl.data_ptr(), want.data_ptr(),
                                     pacc.data_ptr(), pml.data_ptr(), *sizes, 128 ** -0.5, stream)
    _lib.check(rc, "paged_decode_attn")
    rc = lib.mi355_paged_decode_attn_static(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(), sl.data_ptr(),
                                            got.data_ptr(), *sizes, 128 ** -0.5, stream)
    _lib.check(rc, "paged_decode_attn_static")
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_no_alloc_decode_matches_caller_scratch_twice(dev):
    from oracle import inputs, paged_decode as op

    announce("no-alloc decode: 12 seqs x 4 splits, then 5 seqs x 3 splits")
    big = inputs.paged_decode_inputs(num_seqs=12, min_len=40, max_len=2000, seed=31)
    got, want = _both(dev, *big, 4)
    assert torch.equal(got, want)
    torch.testing.assert_close(got.float(), op.paged_decode_ref(*big), rtol=1e-2, atol=2e-3)
    small = inputs.paged_decode_inputs(num_seqs=5, min_len=1, max_len=300, seed=32)
    got, want = _both(dev, *small, 3)
    assert torch.equal(got, want)
    torch.testing.assert_close(got.float(), op.paged_decode_ref(*small), rtol=1e-2, atol=2e-3)
    announce("no-alloc decode: single split (no partials at all)")
    got, want = _both(dev, *small, 1)
    assert torch.equal(got, want)


def test_no_alloc_decode_allocates_nothing(dev):
    """The property in the entry point's name: free device memory (hipMemGetInfo) is the same before and after a
    call once the first call on the device has looked up the array's address."""
    from iree_turbine_amd import _lib
    from oracle import inputs

    lib = _lib.load()
    q, kc, vc, bt, sl = (t.to(dev).contiguous() for t in inputs.paged_decode_inputs(num_seqs=6, min_len=30, max_len=700, seed=33))
    S, Hq, D = q.shape
    P, page, Hkv, _ = kc.shape
    out = torch.empty((S, Hq, D), dtype=torch.float16, device=dev)
    stream = _lib.current_stream_ptr(dev)

    def call():
        rc = lib.mi355_paged_decode_attn_static(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(), sl.data_ptr(),
                                                out.data_ptr(), S, Hq, Hkv, D, page, bt.shape[1], P, 4, 128 ** -0.5, stream)
        _lib.check(rc, "paged_decode_attn_static")
        torch.cuda.synchronize()

    announce("no-alloc decode: free device memory unchanged across calls")
    call()  # the first call on a device may load the code object and looks up the array
    free_before, _ = torch.cuda.mem_get_info(dev)
    for _ in range(3):
        call()
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before


def test_no_alloc_decode_at_the_arrays_last_row(dev):
    """num_seqs x num_q_heads x num_splits == 32768 exactly: the last partial ends at the array's last float."""
    from oracle import inputs

    announce("no-alloc decode: 64 seqs x 32 heads x 16 splits = 32768 rows (the limit)")
    case = inputs.paged_decode_inputs(num_seqs=64, min_len=300, max_len=1200, seed=34)
    got, want = _both(dev, *case, 16)
    assert torch.equal(got, want)


def test_no_alloc_decode_rejects_sizes_beyond_its_array(dev):
    from iree_turbine_amd import _lib

    lib = _lib.load()
    t = torch.zeros(16, dtype=torch.float16, device=dev)
    i = torch.zeros(16, dtype=torch.int32, device=dev)
    # 64 seqs x 32 heads x 17 splits = 34816 rows > 32768: refused before anything is launched or dereferenced
    rc = lib.mi355_paged_decode_attn_static(t.data_ptr(), t.data_ptr(), t.data_ptr(), i.data_ptr(), i.data_ptr(), t.data_ptr(),
                                            64, 32, 8, 128, 16, 512, 1000, 17, 0.088, _lib.current_stream_ptr(dev))
    assert rc == -5 and "exceeds the built-in scratch" in _lib.last_error()
