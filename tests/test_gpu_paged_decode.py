"""GPU parity: paged GQA decode attention through the C ABI vs the CPU oracle (gather + dense fp32)."""

import pytest
import torch

from conftest import announce

pytestmark = pytest.mark.gpu

ATOL = 2e-3
RTOL = 1e-2


def _to(dev, *ts):
    return [t.to(dev) for t in ts]


@pytest.mark.parametrize("splits", [1, 2, 4, 7, 0])
def test_decode_small(dev, splits):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce(f"paged decode small splits={splits}")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=6, min_len=1, max_len=700, seed=4)
    out = torch.ops.mi355.paged_decode_attn(*_to(dev, q, kc, vc, bt, sl), 0.0, splits)
    ref = op.paged_decode_ref(q, kc, vc, bt, sl)
    torch.testing.assert_close(out.float().cpu(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("hq,hkv", [(8, 8), (8, 4), (32, 8), (16, 2), (16, 1)])
def test_decode_gqa_ratios(dev, hq, hkv):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce(f"paged decode hq={hq} hkv={hkv}")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=3, num_q_heads=hq, num_kv_heads=hkv, min_len=5, max_len=300, seed=9)
    out = torch.ops.mi355.paged_decode_attn(*_to(dev, q, kc, vc, bt, sl), 0.0, 2)
    ref = op.paged_decode_ref(q, kc, vc, bt, sl)
    torch.testing.assert_close(out.float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_decode_edge_lengths_and_poison(dev):
    """Lengths around page boundaries; tail tokens of the last page and unused pages hold NaN, padded
    block-table entries hold an out-of-range id: none of them may influence (or be read into) the result."""
    import iree_turbine_amd  # noqa: F401
    from oracle import paged_decode as op

    announce("paged decode edge lengths + poison")
    lens = torch.tensor([1, 15, 16, 17, 31, 32, 33, 160, 161, 0], dtype=torch.int32)
    S, Hq, Hkv, D, page = lens.numel(), 8, 2, 128, 16
    n_pg = (lens + page - 1) // page
    P = int(n_pg.sum()) + 3
    g = torch.Generator().manual_seed(11)
    perm = torch.randperm(P, generator=g)
    bt = torch.full((S, int(n_pg.max()) + 2), 2**30, dtype=torch.int32)
    kc = torch.full((P, page, Hkv, D), float("nan")).half()
    vc = torch.full((P, page, Hkv, D), float("nan")).half()
    off = 0
    for s in range(S):
        n = int(n_pg[s])
        bt[s, :n] = perm[off:off + n].int()
        for i in range(n):
            valid = min(page, int(lens[s]) - i * page)
            pg = int(perm[off + i])
            kc[pg, :valid] = torch.randn(valid, Hkv, D, generator=g).half()
            vc[pg, :valid] = torch.randn(valid, Hkv, D, generator=g).half()
        off += n
    q = torch.randn(S, Hq, D, generator=g).half()
    kz, vz = torch.nan_to_num(kc, nan=0.0), torch.nan_to_num(vc, nan=0.0)
    bt_ref = bt.clone()
    bt_ref[bt_ref == 2**30] = 0
    ref = op.paged_decode_ref(q, kz, vz, bt_ref, lens)
    for splits in (1, 3):
        out = torch.ops.mi355.paged_decode_attn(*_to(dev, q, kc, vc, bt, lens), 0.0, splits).float().cpu()
        assert not torch.isnan(out).any()
        torch.testing.assert_close(out, ref, rtol=RTOL, atol=ATOL)
        assert torch.equal(out[-1], torch.zeros(Hq, D))  # an empty sequence yields zeros


@pytest.mark.parametrize("splits", [1, 3])
def test_decode_bad_page_ids_inside_a_sequence_are_dropped(dev, splits):
    """A stale or padding id (-1, or one past the cache) INSIDE a sequence's live range must not become an address:
    that block contributes nothing, exactly as if its 16 tokens were masked out -- also when it is the first block a
    wave sees, and when every block of a sequence is bad (zeros out)."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs

    announce(f"paged decode bad page ids splits={splits}")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=4, num_q_heads=8, num_kv_heads=2, min_len=200, max_len=400, seed=13)
    P = kc.shape[0]
    bad = bt.clone()
    bad[0, 0], bad[0, 3], bad[1, 1], bad[2, 5] = -1, P, 2**30, -(2**31)
    n3 = (int(sl[3]) + 15) // 16
    bad[3, :n3] = -1
    got = torch.ops.mi355.paged_decode_attn(*_to(dev, q, kc, vc, bad, sl), 0.0, splits).float().cpu()
    assert torch.isfinite(got).all()
    assert torch.equal(got[3], torch.zeros(8, 128))
    # the same attention with the dropped blocks masked out by hand: dense softmax over the remaining tokens
    for s, dropped in ((0, (0, 3)), (1, (1,)), (2, (5,))):
        L = int(sl[s])
        keep = torch.ones(L, dtype=torch.bool)
        for b in dropped:
            keep[b * 16:(b + 1) * 16] = False
        pages = bt[s, :(L + 15) // 16].long()
        k = kc[pages].reshape(-1, 2, 128)[:L][keep].float()
        v = vc[pages].reshape(-1, 2, 128)[:L][keep].float()
        for h in range(8):
            p = torch.softmax((k[:, h // 4] @ q[s, h].float()) * 128 ** -0.5, dim=0)
            torch.testing.assert_close(got[s, h], p @ v[:, h // 4], rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("splits", [1, 3])
def test_decode_lengths_outside_the_table(dev, splits):
    """A length beyond what the block table addresses is cut to the table's reach, a negative one counts as
    empty: the table is never read past its end."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs

    announce(f"paged decode out-of-range lengths splits={splits}")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=4, num_q_heads=8, num_kv_heads=2, min_len=100, max_len=300, seed=8)
    width = bt.shape[1]
    longest = int(sl.argmax())
    wild, tame = sl.clone(), sl.clone()
    wild[longest], tame[longest] = 10 ** 6, int((sl[longest] + 15) // 16 * 16)  # its row of the table is full
    other = (longest + 1) % 4
    wild[other], tame[other] = -7, 0
    assert (int(sl[longest]) + 15) // 16 == width
    got = torch.ops.mi355.paged_decode_attn(*_to(dev, q, kc, vc, bt, wild), 0.0, splits)
    want = torch.ops.mi355.paged_decode_attn(*_to(dev, q, kc, vc, bt, tame), 0.0, splits)
    assert torch.equal(got, want)
    assert torch.equal(got[other].cpu(), torch.zeros(8, 128, dtype=torch.float16))


def test_decode_invariances(dev):
    """Independent of the physical page placement and of the number of splits; phase0 + phase1 == fused."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs

    announce("paged decode invariances")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=5, min_len=100, max_len=1500, seed=21)
    args = _to(dev, q, kc, vc, bt, sl)
    base = torch.ops.mi355.paged_decode_attn(*args, 0.0, 4)
    P = kc.shape[0]
    perm = torch.randperm(P, generator=torch.Generator().manual_seed(1))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(P)
    kc2, vc2 = kc[perm], vc[perm]  # page that was at perm[i] is now at i
    bt2 = torch.where(bt >= 0, inv[bt.clamp(min=0).long()].int(), bt)
    moved = torch.ops.mi355.paged_decode_attn(*_to(dev, q, kc2, vc2, bt2, sl), 0.0, 4)
    assert torch.equal(base, moved)
    for splits in (1, 2, 8, 16):
        o = torch.ops.mi355.paged_decode_attn(*args, 0.0, splits)
        torch.testing.assert_close(o.float(), base.float(), rtol=1e-2, atol=1e-3)
    pacc, pml = torch.ops.mi355.paged_decode_phase0(*args, 0.0, 4)
    two = torch.ops.mi355.paged_decode_phase1(pacc, pml)
    assert torch.equal(two, base)


@pytest.mark.parametrize("num_seqs,splits", [(257, 1), (300, 2), (1000, 1)])
def test_decode_large_batches_walk_sequences_by_length_bucket(dev, num_seqs, splits):
    """Beyond 256 sequences the kernel orders its workgroups by length bucket (a counting pass and two block scans)
    instead of by exact rank: every sequence must still be computed exactly once -- equal lengths, empty sequences
    and one very long sequence among short ones included."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce(f"paged decode {num_seqs} sequences splits={splits}")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=num_seqs, num_q_heads=8, num_kv_heads=2, min_len=1, max_len=90, seed=17)
    sl[5] = 0  # equal lengths are plentiful: up to 1000 draws from 90 values
    out = torch.ops.mi355.paged_decode_attn(*_to(dev, q, kc, vc, bt, sl), 0.0, splits)
    ref = op.paged_decode_ref(q, kc, vc, bt, sl)
    torch.testing.assert_close(out.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    assert torch.equal(out[5].cpu(), torch.zeros(8, 128, dtype=torch.float16))


def test_decode_one_launch_merge_equals_two_phase(dev):
    """The op merges the kv splits inside the phase-0 kernel (the last workgroup of a (sequence, kv head) to finish
    does it); the C entry with caller scratch runs phase 0 and phase 1 as two launches.  Same arithmetic: bit-equal,
    over calls in a row with different split counts, batch shapes and dtypes (the arrival counters must come back
    to zero every time), with a window, and for the full benchmark batch."""
    import iree_turbine_amd  # noqa: F401
    from iree_turbine_amd import _lib, launch
    from oracle import inputs

    lib = _lib.load()

    def two_phase(q, kc, vc, bt, sl, splits):
        S, Hq, D = q.shape
        P, page, Hkv, _ = kc.shape
        out = torch.empty_like(q)
        pacc = torch.empty((S, Hq, splits, D), dtype=torch.float32, device=dev)
        pml = torch.empty((S, Hq, splits, 2), dtype=torch.float32, device=dev)
        entry = lib.mi355_paged_decode_attn_window_bf16 if q.dtype == torch.bfloat16 else lib.mi355_paged_decode_attn_window
        rc = entry(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(), sl.data_ptr(), out.data_ptr(), pacc.data_ptr(),
                   pml.data_ptr(), S, Hq, Hkv, D, page, bt.shape[1], P, splits, 128 ** -0.5, 0, _lib.current_stream_ptr(dev))
        _lib.check(rc, "two-phase decode")
        return out

    cases = [(dict(num_seqs=7, min_len=1, max_len=900, seed=41), 4, False), (dict(num_seqs=3, min_len=300, max_len=2000, seed=42), 9, False),
             (dict(num_seqs=7, min_len=1, max_len=900, seed=43), 2, True), (dict(), 3, False), (dict(num_seqs=2, min_len=50, max_len=60, seed=44), 16, False)]
    for kw, splits, bf in cases:
        announce(f"decode one-launch merge {kw} splits={splits} bf16={bf}")
        q, kc, vc, bt, sl = _to(dev, *inputs.paged_decode_inputs(**kw))
        if bf:
            q, kc, vc = q.bfloat16(), kc.bfloat16(), vc.bfloat16()
        got = torch.ops.mi355.paged_decode_attn(q, kc, vc, bt, sl, 0.0, splits)
        assert torch.equal(got, two_phase(q, kc, vc, bt, sl, splits))
    torch.cuda.synchronize()
    assert launch._ARRIVALS and all(int(buf.abs().sum()) == 0 for buf in launch._ARRIVALS.values())


def test_decode_one_launch_merge_does_not_depend_on_the_counters(dev):
    """The arrival counters are tagged per call: words left behind by a call that never finished, or memory that was
    never cleared, count as zero.  The counters are filled with junk (words whose tag cannot be a live call's: tags
    are at most 2^20 - 1, the junk carries 0xFFFFF) before each of two calls; the result is the two-launch result bit
    for bit and the words the call used are zero afterwards."""
    import iree_turbine_amd  # noqa: F401
    from iree_turbine_amd import _lib
    from oracle import inputs

    announce("decode one-launch merge over junk counters")
    lib = _lib.load()
    q, kc, vc, bt, sl = _to(dev, *inputs.paged_decode_inputs(num_seqs=5, min_len=100, max_len=1500, seed=47))
    S, Hq, D = q.shape
    P, page, Hkv, _ = kc.shape
    splits = 5
    pacc = torch.empty((S, Hq, splits, D), dtype=torch.float32, device=dev)
    pml = torch.empty((S, Hq, splits, 2), dtype=torch.float32, device=dev)
    ref = torch.empty_like(q)
    rc = lib.mi355_paged_decode_attn(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(), sl.data_ptr(), ref.data_ptr(),
                                     pacc.data_ptr(), pml.data_ptr(), S, Hq, Hkv, D, page, bt.shape[1], P, splits, 128 ** -0.5,
                                     _lib.current_stream_ptr(dev))
    _lib.check(rc, "two-launch decode")
    for junk in (0xFFFFF003, 0xFFFFF000 | (splits - 1)):
        counters = torch.full((S * Hkv,), junk - (1 << 32), dtype=torch.int32, device=dev)
        out = torch.full_like(q, 9.0)
        rc = lib.mi355_paged_decode_attn_fused(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(), sl.data_ptr(),
                                               out.data_ptr(), pacc.data_ptr(), pml.data_ptr(), counters.data_ptr(), S, Hq, Hkv, D,
                                               page, bt.shape[1], P, splits, 128 ** -0.5, 0, _lib.dtype_code(torch.float16),
                                               _lib.current_stream_ptr(dev))
        _lib.check(rc, "one-launch decode")
        assert torch.equal(out, ref)
        assert int(counters.abs().sum()) == 0


def test_decode_one_launch_merge_under_graph_replay(dev):
    """The one-launch form captured into a HIP graph (after one eager call, which creates the stream's counters),
    replayed several times with eager calls of other shapes in between, then called eagerly again: every result is
    the two-launch result bit for bit.  A replay reuses its call's tag; it relies on the replay before having left
    its words zero."""
    import iree_turbine_amd  # noqa: F401
    from iree_turbine_amd import _lib, launch
    from oracle import inputs

    announce("decode one-launch merge, graph capture and replays")
    lib = _lib.load()
    q, kc, vc, bt, sl = _to(dev, *inputs.paged_decode_inputs(num_seqs=6, min_len=200, max_len=1800, seed=48))
    q2, kc2, vc2, bt2, sl2 = _to(dev, *inputs.paged_decode_inputs(num_seqs=3, min_len=10, max_len=700, seed=49))
    S, Hq, D = q.shape
    P, page, Hkv, _ = kc.shape
    splits = 4
    pacc = torch.empty((S, Hq, splits, D), dtype=torch.float32, device=dev)
    pml = torch.empty((S, Hq, splits, 2), dtype=torch.float32, device=dev)
    ref = torch.empty_like(q)
    rc = lib.mi355_paged_decode_attn(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(), sl.data_ptr(), ref.data_ptr(),
                                     pacc.data_ptr(), pml.data_ptr(), S, Hq, Hkv, D, page, bt.shape[1], P, splits, 128 ** -0.5,
                                     _lib.current_stream_ptr(dev))
    _lib.check(rc, "two-launch decode")
    side = torch.cuda.Stream(device=dev)  # (default priority)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        out = torch.empty_like(q)
        launch.paged_decode_attn_out(q, kc, vc, bt, sl, out, 0.0, splits)  # eager: creates this stream's counters
        assert torch.equal(out, ref)
        graph = torch.cuda.CUDAGraph()
        out.fill_(3.0)
        with torch.cuda.graph(graph, stream=side):
            launch.paged_decode_attn_out(q, kc, vc, bt, sl, out, 0.0, splits)
        for rep in range(4):  # (the capture above ran on a stream with counters: the one-launch form is what replays)
            out.fill_(float(rep))
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, ref), f"replay {rep}"
            other = torch.ops.mi355.paged_decode_attn(q2, kc2, vc2, bt2, sl2, 0.0, 3)  # eager work between the replays
            torch.cuda.synchronize()
            assert torch.isfinite(other.float()).all()
        out.fill_(5.0)
        launch.paged_decode_attn_out(q, kc, vc, bt, sl, out, 0.0, splits)
        torch.cuda.synchronize()
        assert torch.equal(out, ref)
    torch.cuda.current_stream(dev).wait_stream(side)


def test_decode_full_size(dev):
    """The benchmark configuration (64 seqs, 32/8 heads, ctx in [512, 8192]) against the oracle."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce("paged decode full size")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs()
    out = torch.ops.mi355.paged_decode_attn(*_to(dev, q, kc, vc, bt, sl), 0.0, 0)
    ref = op.paged_decode_ref(q, kc, vc, bt, sl)
    torch.testing.assert_close(out.float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_decode_contract_errors(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs

    q, kc, vc, bt, sl = _to(dev, *inputs.paged_decode_inputs(num_seqs=2, min_len=5, max_len=40))
    with pytest.raises(ValueError):
        torch.ops.mi355.paged_decode_attn(q, kc, vc, bt.long(), sl, 0.0, 1)
    with pytest.raises(ValueError):
        torch.ops.mi355.paged_decode_attn(q, kc[:, :8], vc[:, :8], bt, sl, 0.0, 1)  # page size 8
    with pytest.raises(ValueError):
        torch.ops.mi355.paged_decode_attn(q[:, :3], kc, vc, bt, sl, 0.0, 1)  # 3 q heads over 8 kv heads


@pytest.mark.parametrize("window", [1, 5, 16, 17, 100, 1000, 100000])
@pytest.mark.parametrize("splits", [1, 3])
def test_decode_sliding_window(dev, window, splits):
    """Windows smaller than a page, straddling pages, larger than every sequence; single and split-K."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce(f"paged decode window={window} splits={splits}")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=6, num_q_heads=16, num_kv_heads=4, min_len=1, max_len=700, seed=21)
    out = torch.ops.mi355.paged_decode_attn_window(*_to(dev, q, kc, vc, bt, sl), 0.0, splits, window)
    ref = op.paged_decode_ref(q, kc, vc, bt, sl, window=window)
    torch.testing.assert_close(out.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    if window >= 700:  # the window covers everything: identical to the plain op
        assert torch.equal(out, torch.ops.mi355.paged_decode_attn(*_to(dev, q, kc, vc, bt, sl), 0.0, splits))


def test_decode_window_ignores_tokens_in_front(dev):
    """Tokens in front of the window may hold anything finite: the result does not move."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs

    announce("paged decode window isolation")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=3, num_q_heads=8, num_kv_heads=8, min_len=200, max_len=300, seed=5)
    W = 40
    base = torch.ops.mi355.paged_decode_attn_window(*_to(dev, q, kc, vc, bt, sl), 0.0, 2, W)
    kc2, vc2 = kc.clone(), vc.clone()
    for s in range(3):
        lo = int(sl[s]) - W
        for t in range(lo):  # overwrite everything in front of the window
            kc2[int(bt[s, t // 16]), t % 16] = 7.0
            vc2[int(bt[s, t // 16]), t % 16] = -9.0
    again = torch.ops.mi355.paged_decode_attn_window(*_to(dev, q, kc2, vc2, bt, sl), 0.0, 2, W)
    assert torch.equal(base, again)


@pytest.mark.parametrize("n_new", [1, 5, 40])
def test_kv_cache_append(dev, n_new):
    """Bit-exact against slice assignment through the table; then decode over the appended cache."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce(f"kv_cache_append n_new={n_new}")
    S, Hq, Hkv = 7, 16, 4
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=S, num_q_heads=Hq, num_kv_heads=Hkv, min_len=64, max_len=400, seed=8)
    g = torch.Generator().manual_seed(n_new)
    # the new tokens fill the tail of every sequence (one of them from position 0)
    start = (sl - n_new).clamp(min=0).int()
    start[0] = 0
    kn = torch.randn(S, n_new, Hkv, 128, generator=g).half()
    vn = torch.randn(S, n_new, Hkv, 128, generator=g).half()
    kd, vd = kc.to(dev), vc.to(dev)
    torch.ops.mi355.kv_cache_append(kn.to(dev), vn.to(dev), kd, vd, bt.to(dev), start.to(dev))
    kr, vr = op.kv_cache_append_ref(kn, vn, kc, vc, bt, start)
    assert torch.equal(kd.cpu(), kr) and torch.equal(vd.cpu(), vr)
    assert not torch.equal(kr, kc)
    out = torch.ops.mi355.paged_decode_attn(q.to(dev), kd, vd, bt.to(dev), sl.to(dev), 0.0, 0)
    torch.testing.assert_close(out.float().cpu(), op.paged_decode_ref(q, kr, vr, bt, sl), rtol=RTOL, atol=ATOL)


def test_kv_cache_append_skips_positions_without_a_page(dev):
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce("kv_cache_append bounds")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=4, num_q_heads=8, num_kv_heads=2, min_len=20, max_len=60, seed=2)
    kn = torch.ones(4, 3, 2, 128).half()
    # beyond the table width, into a padded (-1) entry, negative
    start = torch.tensor([16 * bt.shape[1] - 1, int(sl[1] + 15) // 16 * 16, -2, 0], dtype=torch.int32)
    bt2 = bt.clone()
    if int((sl[1] + 15) // 16) < bt.shape[1]:
        assert bt2[1, int((sl[1] + 15) // 16)] == -1
    kd, vd = kc.to(dev), vc.to(dev)
    torch.ops.mi355.kv_cache_append(kn.to(dev), kn.to(dev), kd, vd, bt2.to(dev), start.to(dev))
    kr, vr = op.kv_cache_append_ref(kn, kn, kc, vc, bt2, start)
    assert torch.equal(kd.cpu(), kr) and torch.equal(vd.cpu(), vr)
    with pytest.raises(ValueError):
        torch.ops.mi355.kv_cache_append(kn.to(dev), kn.to(dev), kd, vd, bt2.to(dev), start.long().to(dev))
    with pytest.raises(ValueError):
        torch.ops.mi355.paged_decode_attn_window(*_to(dev, q, kc, vc, bt, sl), 0.0, 1, -1)


@pytest.mark.parametrize("n_new", [1, 16, 100, 200])
@pytest.mark.parametrize("hq,hkv", [(8, 2), (4, 4)])
def test_paged_prefill_vs_oracle(dev, n_new, hq, hkv):
    """Chunked prefill over the paged cache: chunks shorter and longer than a query block, prefixes that end
    inside a page, sequences shorter than the chunk (their first queries see nothing: zeros)."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce(f"paged prefill n_new={n_new} hq={hq} hkv={hkv}")
    _, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=5, num_q_heads=hq, num_kv_heads=hkv, min_len=40, max_len=600, seed=6)
    g = torch.Generator().manual_seed(n_new)
    q = torch.randn(5, n_new, hq, 128, generator=g).half()
    out = torch.ops.mi355.paged_prefill_attn(*_to(dev, q, kc, vc, bt, sl), 0.0)
    torch.cuda.synchronize()
    ref = op.paged_prefill_ref(q, kc, vc, bt, sl)
    torch.testing.assert_close(out.float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_paged_prefill_matches_decode_and_dense_attention(dev):
    """One new token is the decode kernel's problem; a chunk covering the whole sequence on an in-order block
    table is plain causal attention over the same rows."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs

    announce("paged prefill vs decode kernel and dense kernel")
    q1, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=6, num_q_heads=16, num_kv_heads=4, min_len=1, max_len=900, seed=8)
    dq, dkc, dvc, dbt, dsl = _to(dev, q1, kc, vc, bt, sl)
    a = torch.ops.mi355.paged_prefill_attn(dq[:, None].contiguous(), dkc, dvc, dbt, dsl, 0.0)[:, 0]
    b = torch.ops.mi355.paged_decode_attn(dq, dkc, dvc, dbt, dsl, 0.0, 1)
    torch.testing.assert_close(a.float(), b.float(), rtol=RTOL, atol=ATOL)
    # dense: sequence of 320 tokens in pages 0..19, queries for all of them
    S, L, Hq, Hkv = 2, 320, 8, 2
    g = torch.Generator().manual_seed(3)
    k = torch.randn(S, L, Hkv, 128, generator=g).half().to(dev)
    v = torch.randn(S, L, Hkv, 128, generator=g).half().to(dev)
    q = torch.randn(S, L, Hq, 128, generator=g).half().to(dev)
    kcache, vcache = k.reshape(S * L // 16, 16, Hkv, 128), v.reshape(S * L // 16, 16, Hkv, 128)
    table = torch.arange(S * L // 16, dtype=torch.int32, device=dev).reshape(S, L // 16)
    lens = torch.full((S,), L, dtype=torch.int32, device=dev)
    paged = torch.ops.mi355.paged_prefill_attn(q, kcache, vcache, table, lens, 0.0)
    from iree_turbine_amd import launch
    qt = q.transpose(1, 2)
    dense = torch.empty_like(qt)  # laid out like q
    launch.flash_attn_fwd_out(qt, k.transpose(1, 2), v.transpose(1, 2), dense, True, 0.0, 5)  # the four-wave 16x16x32 form the paged kernel is
    assert torch.equal(paged, dense.transpose(1, 2).contiguous())  # same kernel, same tiles, pages in order: bit-identical
    launch.flash_attn_fwd_out(qt, k.transpose(1, 2), v.transpose(1, 2), dense, True, 0.0, 0)  # the 32x32x16 form
    torch.testing.assert_close(paged.float(), dense.transpose(1, 2).float(), rtol=RTOL, atol=ATOL)


def test_paged_prefill_guards(dev):
    """Page ids outside the cache and table entries beyond the sequence are never dereferenced: poisoned
    entries change nothing; contract violations raise."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs

    announce("paged prefill guards")
    _, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=4, num_q_heads=8, num_kv_heads=2, min_len=20, max_len=300, seed=12)
    q = torch.randn(4, 24, 8, 128, generator=torch.Generator().manual_seed(1)).half()
    dq, dkc, dvc, dbt, dsl = _to(dev, q, kc, vc, bt, sl)
    want = torch.ops.mi355.paged_prefill_attn(dq, dkc, dvc, dbt, dsl, 0.0)
    poisoned = dbt.clone()
    for s in range(4):
        used = (int(sl[s]) + 15) // 16
        poisoned[s, used:] = 2 ** 30
    assert torch.equal(torch.ops.mi355.paged_prefill_attn(dq, dkc, dvc, poisoned, dsl, 0.0), want)
    with pytest.raises(ValueError):
        torch.ops.mi355.paged_prefill_attn(dq[..., :64].contiguous(), dkc, dvc, dbt, dsl, 0.0)
    with pytest.raises(ValueError):
        torch.ops.mi355.paged_prefill_attn(dq, dkc, dvc, dbt.long(), dsl, 0.0)


@pytest.mark.parametrize("page", [32, 64, 128, 256])
def test_larger_pages_decode_append_prefill(dev, page):
    """Pages of 32..256 tokens: the kernels walk 16-token blocks inside them.  Decode (with and without split
    and window), append and chunked prefill against the oracles, which gather whole pages."""
    import iree_turbine_amd  # noqa: F401
    from oracle import inputs, paged_decode as op

    announce(f"paged kernels with page size {page}")
    q, kc, vc, bt, sl = inputs.paged_decode_inputs(num_seqs=5, num_q_heads=8, num_kv_heads=2, page=page, min_len=1, max_len=900, seed=13)
    dq, dkc, dvc, dbt, dsl = _to(dev, q, kc, vc, bt, sl)
    for splits in (1, 3):
        out = torch.ops.mi355.paged_decode_attn(dq, dkc, dvc, dbt, dsl, 0.0, splits)
        torch.testing.assert_close(out.float().cpu(), op.paged_decode_ref(q, kc, vc, bt, sl), rtol=RTOL, atol=ATOL)
    out = torch.ops.mi355.paged_decode_attn_window(dq, dkc, dvc, dbt, dsl, 0.0, 2, 100)
    torch.testing.assert_close(out.float().cpu(), op.paged_decode_ref(q, kc, vc, bt, sl, window=100), rtol=RTOL, atol=ATOL)
    # append 40 tokens at the end of every sequence that has room for them in its own pages
    n_new = 40
    g = torch.Generator().manual_seed(page)
    kn = torch.randn(5, n_new, 2, 128, generator=g).half()
    vn = torch.randn(5, n_new, 2, 128, generator=g).half()
    start = (sl - n_new).clamp(min=0).int()
    k2, v2 = dkc.clone(), dvc.clone()
    torch.ops.mi355.kv_cache_append(kn.to(dev), vn.to(dev), k2, v2, dbt, start.to(dev))
    kr, vr = op.kv_cache_append_ref(kn, vn, kc, vc, bt, start)
    assert torch.equal(k2.cpu(), kr) and torch.equal(v2.cpu(), vr)
    # chunked prefill of those 40 tokens over the updated caches
    qn = torch.randn(5, n_new, 8, 128, generator=g).half()
    lens2 = torch.maximum(sl, torch.full_like(sl, n_new)).int()  # sequences shorter than the chunk grew to its length
    ok = [s for s in range(5) if int(lens2[s]) <= int((sl[s] + page - 1) // page) * page]  # ... if their pages hold it
    got = torch.ops.mi355.paged_prefill_attn(qn.to(dev), k2, v2, dbt, lens2.to(dev), 0.0).float().cpu()
    ref = op.paged_prefill_ref(qn, kr, vr, bt, lens2)
    assert len(ok) >= 3
    torch.testing.assert_close(got[ok], ref[ok], rtol=RTOL, atol=ATOL)
