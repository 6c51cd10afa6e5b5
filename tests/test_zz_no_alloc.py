"""alamd_reduce_scatterv_noalloc against alamd_reduce_scatterv, through the C ABI: the same bits,
on two calls in a row (the second smaller, so what the first left in the fixed scratch array must
not matter), also after other work has used the device; the stated limit is an error."""
import numpy as np
import pytest

import oracle
from util import assert_bits_equal, dev_empty, to_dev, to_host

pytestmark = pytest.mark.gpu

# (P, counts): in-place blocks that overlap their own input at a small displacement (one chained
# launch each), at a displacement of a few runs, and blocks that do not overlap at all
SHAPES = [(3, [1, 3_000_017, 5]), (2, [1, 40_003]), (4, [3, 900_001, 0, 20_000]), (3, [70_000, 100_000, 9]),
          (2, [64, 64])]


def both_ways(al, P, counts, dtype, op, order, seed):
    import torch
    total = sum(counts)
    dist = "fullrange" if dtype[0] in "iu" else "uniform_pm1"
    sends = [oracle.fill(total, dtype, dist, seed + r) for r in range(P)]
    np_dt = sends[0].dtype
    ref = [to_dev(a) for a in sends]
    al.reduce_scatterv(ref, ref, counts, op, order=order, dtype=dtype)
    got = [to_dev(a) for a in sends]
    al.reduce_scatterv_noalloc(got, got, counts, op, order=order, dtype=dtype)
    torch.cuda.synchronize()
    want = oracle.reduce_scatterv(sends, counts, dtype, op, order)
    for b in range(P):
        g, r = to_host(got[b], np_dt), to_host(ref[b], np_dt)
        assert_bits_equal(g[:counts[b]], r[:counts[b]], dtype, "noalloc vs alamd_reduce_scatterv, rank %d" % b)
        assert_bits_equal(g[:counts[b]], want[b], dtype, "noalloc vs oracle, rank %d" % b)
        assert g[counts[b]:].tobytes() == sends[b][counts[b]:].tobytes(), "bytes behind the result changed"
    # separate receive buffers take no scratch at all
    recvs = [dev_empty(max(c, 1), np_dt) for c in counts]
    al.reduce_scatterv_noalloc(recvs, [to_dev(a) for a in sends], counts, op, order=order, dtype=dtype)
    torch.cuda.synchronize()
    for b in range(P):
        assert_bits_equal(to_host(recvs[b], np_dt)[:counts[b]], want[b], dtype, "noalloc, separate buffers, rank %d" % b)


@pytest.mark.parametrize("dtype,op,order", [("f32", "sum", "rank_asc"), ("bf16", "sum", "tree_halv"),
                                            ("i16", "max", "rank_asc"), ("f64", "avg", "pairwise_desc")])
def test_noalloc_two_calls_in_a_row(al, dtype, op, order):
    for k, (P, counts) in enumerate(SHAPES):  # every call after the first is smaller or of another shape
        both_ways(al, P, counts, dtype, op, order, 500 + 10 * k)


def test_noalloc_limit_is_an_error(al):
    import torch
    # an in-place block that overlaps its own input and is longer than the fixed array covers
    limit = ((1 << 20) - 256) // 4 * 4096
    counts = [1, limit + 4096]
    bufs = [torch.zeros(sum(counts), dtype=torch.uint8, device="cuda") for _ in range(2)]
    with pytest.raises(al.AlError, match="beyond the .* bytes the fixed scratch covers") as e:
        al.reduce_scatterv_noalloc(bufs, bufs, counts, "bor", dtype="u8")
    assert e.value.code == 1
    torch.cuda.synchronize()
    # the same block through separate receive buffers has no limit
    recvs = [torch.zeros(c, dtype=torch.uint8, device="cuda") for c in counts]
    al.reduce_scatterv_noalloc(recvs, bufs, counts, "bor", dtype="u8")
    torch.cuda.synchronize()
    assert int(recvs[1].max()) == 0
    del recvs, bufs
    # as long a block that starts a 16th of its length into its buffer: plain launches stand in for the chain
    counts = [(limit + 4096) // 16, limit + 4096]
    gen = torch.Generator(device="cuda").manual_seed(5)
    bufs = [torch.randint(0, 256, (sum(counts),), dtype=torch.uint8, device="cuda", generator=gen) for _ in range(2)]
    want = [bufs[0][:counts[0]] | bufs[1][:counts[0]], bufs[0][counts[0]:] | bufs[1][counts[0]:]]
    al.reduce_scatterv_noalloc(bufs, bufs, counts, "bor", dtype="u8")
    torch.cuda.synchronize()
    for b in range(2):
        assert torch.equal(bufs[b][:counts[b]], want[b]), "long in-place block, rank %d" % b


def test_noalloc_in_a_hip_graph(al):
    """What the entry point is for: an in-place Reduce_scatterv whose block overlaps its own input,
    captured into a HIP graph (no allocation may happen under capture; the scratch is cleared by a
    kernel).  Every replay, with fresh inputs and eager work in between, gives the oracle's bits."""
    import torch
    P, counts = 3, [1, 2_000_003, 7]
    total = sum(counts)
    src = [dev_empty(total, np.float32) for _ in range(P)]
    work = [dev_empty(total, np.float32) for _ in range(P)]

    def run():
        for r in range(P):
            al.copy(work[r], src[r])
        al.reduce_scatterv_noalloc(work, work, counts, "sum", order="tree_halv", dtype="f32")

    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        run()  # no eager call beforehand: the entry point needs no warm-up
    for rep in range(3):
        fresh = [oracle.fill(total, "f32", "uniform_pm1", 700 + 10 * rep + r) for r in range(P)]
        for t, a in zip(src, fresh):
            t.copy_(torch.from_numpy(a))  # eager work between the replays
        for t in work:
            t.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = oracle.reduce_scatterv(fresh, counts, "f32", "sum", "tree_halv")
        for b in range(P):
            got = to_host(work[b], np.float32)
            assert_bits_equal(got[:counts[b]], want[b], "f32", "graph replay %d rank %d" % (rep, b))
            assert got[counts[b]:].tobytes() == fresh[b][counts[b]:].tobytes(), "bytes behind the result changed"


def test_noalloc_refuses_a_second_stream_while_the_array_is_in_use(al):
    """Every call on a device shares the one fixed array.  A chained launch is held back on its stream by a
    flag that the host has not signalled yet; a call on another stream that would need the array meanwhile
    is refused; once the first has run, the second stream's call goes through and is right."""
    import torch
    P, counts = 2, [1, 300_001]
    total = sum(counts)
    sends = [oracle.fill(total, "f32", "uniform_pm1", 40 + r) for r in range(P)]
    want = oracle.reduce_scatterv(sends, counts, "f32", "sum", "rank_asc")
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    first = [to_dev(x) for x in sends]
    second = [to_dev(x) for x in sends]
    torch.cuda.synchronize()
    flag = al.Flag(0)
    try:
        flag.wait(1, mode="kernel", max_spins=1 << 34, stream=a)  # bounded: the stream goes on by itself in the end
        al.reduce_scatterv_noalloc(first, first, counts, "sum", dtype="f32", stream=a)
        with pytest.raises(al.AlError, match="still in use") as e:
            al.reduce_scatterv_noalloc(second, second, counts, "sum", dtype="f32", stream=b)
        assert e.value.code == 1
        # the same stream may queue another one behind its own
        al.reduce_scatterv_noalloc(first, first, [1, 1000], "sum", dtype="f32", stream=a)
    finally:
        flag.signal(1)
    a.synchronize()
    assert not flag.timed_out()
    second = [to_dev(x) for x in sends]
    al.reduce_scatterv_noalloc(second, second, counts, "sum", dtype="f32", stream=b)
    torch.cuda.synchronize()
    for r in range(P):
        assert_bits_equal(to_host(second[r], np.float32)[:counts[r]], want[r], "f32", "second stream, rank %d" % r)
    flag.destroy()
