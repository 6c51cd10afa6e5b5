"""GPU parity of alamd_combine / reduce_scatter / allgather against the CPU
oracle, through the C ABI.  Bit-exact for every type; two NaNs compare equal
whatever their payload."""
import numpy as np
import pytest

import oracle
from util import (ALL_DTYPES, FLOAT_DTYPES, INT_DTYPES, ORDERS, assert_bits_equal, dev_empty, planted_specials,
                  ops_of, to_dev, to_host)

pytestmark = pytest.mark.gpu

DIST_FOR = {"sum": "uniform_pm1", "prod": "uniform_09_11", "min": "uniform_pm1", "max": "uniform_pm1",
            "lor": "bool01", "land": "bool01", "lxor": "bool01", "bor": "fullrange",
            "band": "fullrange", "bxor": "fullrange", "avg": "uniform_pm1"}


def make_inputs(P, n, dtype, op, seed=1000):
    dist = DIST_FOR[op]
    if dtype in INT_DTYPES and op in ("sum", "prod", "min", "max", "avg"):
        dist = "fullrange"
    return [oracle.fill(n, dtype, dist, seed + r) for r in range(P)]


def run_combine(al, ins, dtype, op, order, start=0, nout=1):
    import torch
    d_ins = [to_dev(a) for a in ins]
    outs = [dev_empty(ins[0].size, ins[0].dtype) for _ in range(nout)]
    al.combine(outs, d_ins, op, order=order, start=start, dtype=dtype, count=ins[0].size)
    torch.cuda.synchronize()
    return [to_host(o, ins[0].dtype) for o in outs]


@pytest.fixture(params=["shape by size", "block shape"])
def shape(request, al):
    """Runs a test twice: with the launch shapes the library picks by size (the streaming shape at the
    sizes of these tests) and with every fold / tree launch in the block shape."""
    if request.param == "block shape":
        al.tune("block_shape_from_bytes", 1)
        al.tune("block_shape_below_bytes", 1 << 60)
    yield request.param
    al.tune("block_shape_from_bytes", 0)
    al.tune("block_shape_below_bytes", 0)


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_combine_all_ops_orders(al, dtype, shape):
    for op in ops_of(dtype):
        for P in (1, 2, 3, 5, 8):
            orders = ORDERS if dtype in FLOAT_DTYPES else ("rank_asc", "tree_halv")
            for order in orders:
                for n in (1, 37, 4099):
                    start = (P - 1) // 2 if order in ("pairwise_desc", "ring") else 0
                    ins = make_inputs(P, n, dtype, op)
                    want = oracle.combine(ins, dtype, op, order, start)
                    got = run_combine(al, ins, dtype, op, order, start)[0]
                    assert_bits_equal(got, want, dtype, "%s %s P=%d %s n=%d" % (dtype, op, P, order, n))


@pytest.mark.parametrize("dtype", ("u8", "i8", "u16", "i16", "i32"))
def test_logical_operators_on_any_values(al, dtype, shape):
    """lor / land / lxor see an element as true iff it is nonzero, whatever its value, and give 0 or 1; one
    rank alone gets its input back as it is.  (The 8- and 16-bit kernels make the running result 0 / 1 once
    and then only look at the stream each step adds.)"""
    for P in (1, 2, 3, 8, 13):
        for n in (5, 4099, 70001):
            ins = [oracle.fill(n, dtype, "fullrange", 500 + r) for r in range(P)]
            for a in ins[::2]:
                a[::3] = 0  # enough zeros for land and lxor to give both answers
            for op in ("lor", "land", "lxor"):
                want = oracle.combine(ins, dtype, op, "rank_asc")
                got = run_combine(al, ins, dtype, op, "rank_asc")[0]
                assert_bits_equal(got, want, dtype, "%s %s P=%d n=%d" % (dtype, op, P, n))
                if P == 1:
                    assert got.tobytes() == ins[0].tobytes()


@pytest.mark.parametrize("dtype", ("f32", "bf16", "i32"))
@pytest.mark.parametrize("P", (4, 6, 7, 8, 13, 16, 31, 32, 33, 40, 48, 63, 64))
def test_combine_many_ranks(al, dtype, P, shape):
    n = 5000
    for order in ORDERS:
        ins = make_inputs(P, n, dtype, "sum")
        start = P // 3 if order in ("pairwise_desc", "ring") else 0
        want = oracle.combine(ins, dtype, "sum", order, start)
        got = run_combine(al, ins, dtype, "sum", order, start)[0]
        assert_bits_equal(got, want, dtype, "%s P=%d %s" % (dtype, P, order))


def test_combine_64_ranks_fold(al):
    ins = make_inputs(64, 3001, "f32", "sum")
    for order, start in (("rank_asc", 0), ("ring", 17), ("pairwise_desc", 40)):
        want = oracle.combine(ins, "f32", "sum", order, start)
        got = run_combine(al, ins, "f32", "sum", order, start)[0]
        assert_bits_equal(got, want, "f32", order)


def test_combine_allreduce_outputs_and_inplace(al):
    import torch
    P, n = 8, 100003
    ins = make_inputs(P, n, "f32", "sum")
    want = oracle.combine(ins, "f32", "sum", "tree_dbl")
    outs = run_combine(al, ins, "f32", "sum", "tree_dbl", nout=P)
    for o in outs:
        assert_bits_equal(o, want, "f32", "allreduce outputs")
    # in place: every rank's buffer is both its contribution and its result
    bufs = [to_dev(a) for a in ins]
    al.combine(bufs, bufs, "sum", order="tree_dbl")
    torch.cuda.synchronize()
    for b in bufs:
        assert_bits_equal(to_host(b, np.float32), want, "f32", "in-place allreduce")


def test_combine_unaligned_pointers(al):
    import torch
    P, n = 4, 10007
    ins = make_inputs(P, n, "f32", "sum")
    want = oracle.combine(ins, "f32", "sum", "rank_asc")
    base = [to_dev(np.concatenate([np.zeros(1, np.float32), a])) for a in ins]
    views = [b[1:] for b in base]  # 4-byte aligned only
    out = dev_empty(n + 1, np.float32)
    al.combine([out[1:]], views, "sum", dtype="f32", count=n)
    torch.cuda.synchronize()
    assert_bits_equal(to_host(out, np.float32)[1:], want, "f32", "unaligned")


def _offset_view(a, off):
    """Device copy of `a` that starts `off` elements into its allocation."""
    pad = np.zeros(off, a.dtype)
    return to_dev(np.concatenate([pad, a]))[off:]


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_vector_path_at_any_element_alignment(al, dtype, shape):
    """Buffers that are only element-aligned (each input and the output at its own offset) go through the
    128-bit kernels: several tiles plus a ragged tail, fold and tree orders, two outputs."""
    import torch
    P, n = 5, 3 * 4096 + 37
    op = "sum"
    ins = make_inputs(P, n, dtype, op)
    views = [_offset_view(a, 1 + (r % 3)) for r, a in enumerate(ins)]
    for order in ("rank_asc", "tree_dbl"):
        want = oracle.combine(ins, dtype, op, order)
        outs = [dev_empty(n + 3, ins[0].dtype)[3:], dev_empty(n + 2, ins[0].dtype)[2:]]
        al.combine(outs, views, op, order=order, dtype=dtype, count=n)
        torch.cuda.synchronize()
        for o in outs:
            assert_bits_equal(to_host(o, ins[0].dtype), want, dtype, "%s %s" % (dtype, order))


@pytest.mark.parametrize("dtype", ("u8", "i16", "bf16", "f32", "f64"))
def test_head_up_to_the_outputs_64_byte_boundary(al, dtype, shape):
    """The kernels walk the leading elements one by one until the output reaches a 64-byte boundary:
    outputs 1 element to 60 bytes past a boundary, inputs at the same or at other offsets, counts
    shorter than the head, equal to it and far beyond; fold and tree orders, combine and allgather."""
    import torch
    P = 3
    es = oracle.dtype_size(dtype)
    for out_off in (1, 60 // es, max(1, 36 // es)):
        for in_off in (out_off, 0, out_off + 4 // min(es, 4)):
            for n in (1, 64 // es - out_off, 64 // es, 3 * 4096 + 5):
                if n < 1:
                    continue
                ins = make_inputs(P, n, dtype, "sum", seed=90 + out_off)
                views = [_offset_view(a, in_off) for a in ins]
                for order in ("rank_asc", "tree_halv"):
                    want = oracle.combine(ins, dtype, "sum", order)
                    raw = dev_empty(n + out_off + 16, ins[0].dtype)
                    al.combine([raw[out_off:out_off + n]], views, "sum", order=order, dtype=dtype, count=n)
                    torch.cuda.synchronize()
                    assert_bits_equal(to_host(raw, ins[0].dtype)[out_off:out_off + n], want, dtype,
                                      "%s %s out+%d in+%d n=%d" % (dtype, order, out_off, in_off, n))
                recvs = [dev_empty(P * n + out_off + 16, ins[0].dtype) for _ in range(P)]
                al.allgather([r[out_off:out_off + P * n] for r in recvs], views, dtype=dtype, count=n)
                torch.cuda.synchronize()
                for r in recvs:
                    got = to_host(r, ins[0].dtype)[out_off:out_off + P * n]
                    assert got.tobytes() == np.concatenate(ins).tobytes(), "allgather out+%d n=%d" % (out_off, n)


@pytest.mark.parametrize("dtype", ("u8", "bf16", "f32", "f64"))
def test_head_up_to_the_first_inputs_1kib_boundary(al, dtype, shape):
    """From 64 KiB per segment on, the streaming kernels walk the leading elements one by one until the
    first input reaches a 1 KiB boundary (up to 1023 bytes' worth, spread over the segment's first
    workgroups): lengths just below, at and above that size, inputs and outputs at the same and at
    different offsets from one element to one short of 1 KiB, fold and tree orders, two outputs, one
    launch and many; float min under a reduce-scatter + gather order, whose operand roles change from
    block to block, heads included; the ragged segments of a Reduce_scatterv."""
    import torch
    P = 3
    es = oracle.dtype_size(dtype)
    kib = 1024 // es
    for in_off, out_off in ((1, 1), (kib - 1, kib - 1), (kib // 2 + 1, 3), (0, 5), (7, 0)):
        for n in (64 * kib - 1, 64 * kib, 64 * kib + 1, 300 * kib + 37):
            ins = make_inputs(P, n, dtype, "sum", seed=70 + in_off)
            views = [_offset_view(a, in_off + (r if in_off != out_off else 0)) for r, a in enumerate(ins)]
            for order, launch_bytes in (("rank_asc", 0), ("tree_dbl", 0), ("rank_asc", 1 << 18), ("tree_halv", 1 << 18)):
                want = oracle.combine(ins, dtype, "sum", order)
                raws = [dev_empty(n + out_off + 16, ins[0].dtype) for _ in range(2)]
                try:
                    al.tune("launch_bytes", launch_bytes)
                    al.combine([r[out_off:out_off + n] for r in raws], views, "sum", order=order, dtype=dtype, count=n)
                    torch.cuda.synchronize()
                finally:
                    al.tune("launch_bytes", 0)
                for r in raws:
                    assert_bits_equal(to_host(r, ins[0].dtype)[out_off:out_off + n], want, dtype,
                                      "%s %s out+%d in+%d n=%d launches of %d" % (dtype, order, out_off, in_off, n, launch_bytes))
    if dtype in ("bf16", "f32", "f64"):
        n = 200 * kib + 11
        ins = [planted_specials(n, dtype, r) for r in range(5)]
        views = [_offset_view(a, 3) for a in ins]
        for order in ("tree_rsg", "tree_rsg_spread", "rank_asc"):
            want = oracle.combine(ins, dtype, "min", order)
            raw = dev_empty(n + 3, ins[0].dtype)
            al.combine([raw[3:]], views, "min", order=order, dtype=dtype, count=n)
            torch.cuda.synchronize()
            assert_bits_equal(to_host(raw, ins[0].dtype)[3:], want, dtype, "%s min %s, buffers 3 elements in" % (dtype, order))
    counts = [70 * kib + 3, 0, 65 * kib + 1, 5, 129 * kib - 7]
    sends = make_inputs(len(counts), sum(counts), dtype, "sum", seed=77)
    d_sends = [_offset_view(a, 1) for a in sends]
    for order in ("rank_asc", "tree_halv"):
        want = oracle.reduce_scatterv(sends, counts, dtype, "sum", order)
        recvs = [dev_empty(c + 2, sends[0].dtype)[2:] for c in counts]
        al.reduce_scatterv(recvs, d_sends, counts, "sum", order=order, dtype=dtype)
        torch.cuda.synchronize()
        for b, c in enumerate(counts):
            assert_bits_equal(to_host(recvs[b], sends[0].dtype)[:c], want[b], dtype, "reduce_scatterv %s rank %d" % (order, b))


@pytest.mark.parametrize("dtype", ("u8", "bf16", "f32", "f64"))
@pytest.mark.parametrize("inplace", (False, True))
def test_reduce_scatter_odd_block_sizes(al, dtype, inplace):
    """Block sizes that put every block but the first off a 16-byte boundary."""
    import torch
    P = 4
    for count in (1, 7, 4099, 70001):
        op, order = "sum", "pairwise_desc"
        sends = make_inputs(P, P * count, dtype, op, seed=40)
        want = oracle.reduce_scatter(sends, dtype, op, order)
        d_sends = [to_dev(a) for a in sends]
        d_recvs = d_sends if inplace else [dev_empty(count, sends[0].dtype) for _ in range(P)]
        al.reduce_scatter(d_recvs, d_sends, op, order=order, dtype=dtype, count=count)
        torch.cuda.synchronize()
        for r in range(P):
            assert_bits_equal(to_host(d_recvs[r], sends[0].dtype)[:count], want[r], dtype,
                              "%s count=%d rank %d" % (dtype, count, r))


@pytest.mark.parametrize("dtype", ("f32", "f64", "bf16", "f16"))
def test_combine_special_values(al, dtype, shape):
    # NaN, infinities, signed zeros, denormals and ties on every side
    f32 = np.array([np.nan, -1.0, np.nan, 0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-45, 1.0,
                    3.4028235e38, 1.1754944e-38, 0.0, -0.0, np.inf, 5.877472e-39, 65504.0, 1e-8],
                   dtype=np.float32)
    rng = np.random.default_rng(7)
    P = 4
    cols = [f32[rng.permutation(f32.size)] for _ in range(P)]
    # every pair of specials meets somewhere
    grid = [np.concatenate([np.repeat(f32, f32.size), c]) if r == 0 else
            np.concatenate([np.tile(f32, f32.size), c]) if r == 1 else
            np.concatenate([np.full(f32.size ** 2, f32[(3 * r) % f32.size], np.float32), c])
            for r, c in enumerate(cols)]
    if dtype == "f32":
        ins = grid
    elif dtype == "f64":
        ins = [g.astype(np.float64) for g in grid]
    elif dtype == "bf16":
        ins = [oracle.f32_to_bf16(g) for g in grid]
    else:
        ins = [oracle.f32_to_f16(g) for g in grid]
    for op in ("sum", "prod", "min", "max"):
        for order, start in (("rank_asc", 0), ("tree_dbl", 0), ("tree_halv", 0), ("ring", 1),
                             ("pairwise_desc", 2), ("tree_binomial", 0)):
            want = oracle.combine(ins, dtype, op, order, start)
            got = run_combine(al, ins, dtype, op, order, start)[0]
            assert_bits_equal(got, want, dtype, "%s %s %s" % (dtype, op, order))


@pytest.mark.parametrize("P", (3, 5, 8, 12, 16, 33, 48, 64))
def test_float_min_max_operand_roles_over_many_tiles(al, P, shape):
    """Zeros of both signs and NaNs in every operand position (the inputs of the golden vectors' special
    cases), over messages of many tiles whose blocks end inside tiles and whose length is no multiple of
    the power of two of ranks: which operand of every pair lets a tie through depends on the order, the
    start and, under the reduce-scatter + gather orders, on the block the element lies in."""
    import torch
    for dtype, n in (("f32", 70001), ("bf16", 33333), ("f64", 20011)):
        ins = [planted_specials(n, dtype, r) for r in range(P)]
        d_ins = [to_dev(a) for a in ins]
        for op in ("min", "max"):
            for order, start in (("tree_rsg", 0), ("tree_rsg_spread", 0), ("tree_halv", 0), ("tree_halv", P - 1),
                                 ("tree_halv", P // 2), ("tree_binomial", P // 3), ("tree_dbl", 0)):
                want = oracle.combine(ins, dtype, op, order, start)
                outs = [dev_empty(n, ins[0].dtype) for _ in range(2)]
                al.combine(outs, d_ins, op, order=order, start=start, dtype=dtype, count=n)
                torch.cuda.synchronize()
                for o in outs:
                    assert_bits_equal(to_host(o, ins[0].dtype), want, dtype, "%s %s P=%d %s start %d" % (dtype, op, P, order, start))
    # ... and a reduce-scatter, whose tree orders take the receiving rank as start block by block
    count = 1031
    sends = [planted_specials(P * count, "f32", r) for r in range(P)]
    d_sends = [to_dev(a) for a in sends]
    for order in ("tree_halv", "tree_rsg", "tree_rsg_spread"):
        want = oracle.reduce_scatter(sends, "f32", "min", order)
        recvs = [dev_empty(count, np.float32) for _ in range(P)]
        al.reduce_scatter(recvs, d_sends, "min", order=order, dtype="f32", count=count)
        torch.cuda.synchronize()
        for r in range(P):
            assert_bits_equal(to_host(recvs[r], np.float32), want[r], "f32", "reduce_scatter min P=%d %s rank %d" % (P, order, r))


@pytest.mark.parametrize("dtype", ("f32", "bf16", "u8", "i64"))
@pytest.mark.parametrize("order", ("rank_asc", "tree_halv", "pairwise_desc", "ring"))
def test_reduce_scatter(al, dtype, order, shape):
    import torch
    for P in (1, 2, 5, 8):
        for count in (1, 24, 1000, 4096):
            sends = make_inputs(P, P * count, dtype, "sum")
            want = oracle.reduce_scatter(sends, dtype, "sum", order)
            d_sends = [to_dev(a) for a in sends]
            recvs = [dev_empty(count, sends[0].dtype) for _ in range(P)]
            al.reduce_scatter(recvs, d_sends, "sum", order=order, dtype=dtype, count=count)
            torch.cuda.synchronize()
            for r in range(P):
                assert_bits_equal(to_host(recvs[r], sends[0].dtype), want[r], dtype,
                                  "reduce_scatter %s P=%d count=%d rank %d" % (order, P, count, r))
            # in place: the result replaces the start of each send buffer
            al.reduce_scatter(d_sends, d_sends, "sum", order=order, dtype=dtype, count=count)
            torch.cuda.synchronize()
            for r in range(P):
                assert_bits_equal(to_host(d_sends[r], sends[0].dtype)[:count], want[r], dtype,
                                  "in-place reduce_scatter %s P=%d count=%d rank %d" % (order, P, count, r))


@pytest.mark.parametrize("dtype", ("u8", "bf16", "f32", "f64"))
def test_allgather(al, dtype):
    import torch
    for P in (1, 3, 8):
        for count in (1, 5, 1024, 4099):
            sends = make_inputs(P, count, dtype, "bxor" if dtype == "u8" else "sum")
            want = oracle.allgather(sends, dtype)
            d_sends = [to_dev(a) for a in sends]
            recvs = [dev_empty(count * P, sends[0].dtype) for _ in range(P)]
            al.allgather(recvs, d_sends, dtype=dtype, count=count)
            torch.cuda.synchronize()
            for r in range(P):
                assert_bits_equal(to_host(recvs[r], sends[0].dtype), want[r], dtype, "allgather")
            # in place: each rank's slice already sits at its rank offset
            bufs = [to_dev(np.zeros(count * P, sends[0].dtype)) for _ in range(P)]
            for r in range(P):
                bufs[r][r * count:(r + 1) * count].copy_(d_sends[r])
            views = [bufs[r][r * count:(r + 1) * count] for r in range(P)]
            al.allgather(bufs, views, dtype=dtype, count=count)
            torch.cuda.synchronize()
            for r in range(P):
                assert_bits_equal(to_host(bufs[r], sends[0].dtype), want[r], dtype, "in-place allgather")


@pytest.mark.parametrize("dtype", ("f32", "bf16", "i16", "f64"))
@pytest.mark.parametrize("order", ("rank_asc", "tree_halv", "pairwise_desc"))
def test_reduce_scatterv(al, dtype, order, shape):
    import torch
    for P, counts in ((1, [9]), (3, [5, 0, 12]), (4, [1, 100, 3, 64]), (8, [4096, 8, 0, 1000, 8192, 1, 33, 4100])):
        total = sum(counts)
        sends = make_inputs(P, total, dtype, "sum")
        want = oracle.reduce_scatterv(sends, counts, dtype, "sum", order)
        d_sends = [to_dev(a) for a in sends]
        recvs = [dev_empty(max(c, 1), sends[0].dtype) for c in counts]
        al.reduce_scatterv(recvs, d_sends, counts, "sum", order=order, dtype=dtype)
        torch.cuda.synchronize()
        for b in range(P):
            assert_bits_equal(to_host(recvs[b], sends[0].dtype)[:counts[b]], want[b], dtype,
                              "reduce_scatterv %s P=%d rank %d" % (order, P, b))
        # in place: the result replaces the start of each send buffer, also where a rank's own
        # block starts inside the region its result overwrites (counts [1, 100, ...])
        al.reduce_scatterv(d_sends, d_sends, counts, "sum", order=order, dtype=dtype)
        torch.cuda.synchronize()
        for b in range(P):
            assert_bits_equal(to_host(d_sends[b], sends[0].dtype)[:counts[b]], want[b], dtype,
                              "in-place reduce_scatterv %s P=%d rank %d" % (order, P, b))


@pytest.mark.parametrize("dtype,order", [("f32", "rank_asc"), ("f32", "tree_halv"), ("bf16", "pairwise_desc"),
                                         ("f64", "tree_dbl"), ("f16", "tree_binomial"), ("u8", "rank_asc"),
                                         ("i64", "rank_asc"), ("f32", "ring")])
def test_reduce_scatterv_in_place_block_overlapping_its_own_input(al, dtype, order):
    """In place, a block that starts fewer elements into its own buffer than it is long is read and
    overwritten by the same launch at a displacement (any counts are legal:
    include/aluminum/ht/reduce_scatterv.hpp:40-87).  Displacements of one element, of less than a tile,
    of several tiles and a half; lengths with and without a tail; everything behind a rank's result
    stays as it was."""
    import torch
    shapes = [(3, [1, 1_000_003, 5]), (2, [1, 10_000_000]), (4, [3, 200_001, 17, 70_000]),
              (5, [4097, 9 * 4096 + 5, 0, 150_000, 31]), (3, [100_000, 150_000, 400_000]),
              (2, [16, 1 << 20]), (6, [7, 7, 7, 300_000, 1, 2_000_000])]
    if order in ("tree_halv", "tree_dbl", "tree_binomial"):
        shapes.append((40, [2] + [50_000 + 13 * k for k in range(39)]))
    for P, counts in shapes:
        total = sum(counts)
        sends = make_inputs(P, total, dtype, "sum")
        want = oracle.reduce_scatterv(sends, counts, dtype, "sum", order)
        bufs = [to_dev(a) for a in sends]
        al.reduce_scatterv(bufs, bufs, counts, "sum", order=order, dtype=dtype)
        torch.cuda.synchronize()
        for b in range(P):
            got = to_host(bufs[b], sends[0].dtype)
            assert_bits_equal(got[:counts[b]], want[b], dtype, "in place %s %s counts %s rank %d" % (dtype, order, counts[:4], b))
            assert got[counts[b]:].tobytes() == sends[b][counts[b]:].tobytes(), "rank %d: bytes behind the result changed" % b
        # some ranks in place, the others not
        bufs = [to_dev(a) for a in sends]
        recvs = [bufs[b] if b % 2 else dev_empty(max(counts[b], 1), sends[0].dtype) for b in range(P)]
        al.reduce_scatterv(recvs, bufs, counts, "sum", order=order, dtype=dtype)
        torch.cuda.synchronize()
        for b in range(P):
            assert_bits_equal(to_host(recvs[b], sends[0].dtype)[:counts[b]], want[b], dtype, "mixed in place rank %d" % b)


@pytest.mark.parametrize("dtype", ("u8", "i16", "f32", "f64"))
def test_allgatherv(al, dtype):
    import torch
    np_dt = oracle.NP_CARRIER[dtype]
    for P, counts, displs in ((1, [5], [2]), (3, [4, 0, 9], [9, 0, 0]), (4, [1000, 3, 64, 4099], [8, 5400, 1100, 1200]),
                              (8, [16] * 8, [16 * (7 - q) for q in range(8)])):
        sends = [oracle.fill(max(c, 1), dtype, "fullrange" if dtype in ("u8", "i16") else "uniform_pm1", 9 + q)[:c]
                 for q, c in enumerate(counts)]
        want = oracle.allgatherv(sends, counts, displs, dtype, fill_value=0)
        extent = want[0].size
        d_sends = [to_dev(a) if a.size else dev_empty(1, np_dt) for a in sends]
        recvs = [to_dev(np.zeros(extent, np_dt)) for _ in range(P)]
        al.allgatherv(recvs, d_sends, counts, displs, dtype=dtype)
        torch.cuda.synchronize()
        for r in range(P):
            assert_bits_equal(to_host(recvs[r], np_dt), want[r], dtype, "allgatherv P=%d rank %d" % (P, r))
        # in place: each rank's slice already sits at its displacement
        bufs = [to_dev(np.zeros(extent, np_dt)) for _ in range(P)]
        views = []
        for q in range(P):
            v = bufs[q][displs[q]:displs[q] + counts[q]]
            if counts[q]:
                v.copy_(d_sends[q][:counts[q]])
            views.append(v if counts[q] else d_sends[q])
        al.allgatherv(bufs, views, counts, displs, dtype=dtype)
        torch.cuda.synchronize()
        for r in range(P):
            assert_bits_equal(to_host(bufs[r], np_dt), want[r], dtype, "in-place allgatherv P=%d rank %d" % (P, r))
    with pytest.raises(al.AlError) as e:  # slices 0 and 1 collide in the receive buffer
        al.allgatherv(recvs, d_sends, counts, [0, 8] + [100 + 16 * q for q in range(6)], dtype=dtype)
    assert e.value.code == 5


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_avg_division_every_rank_count(al, dtype, shape):
    """avg ends with one division by P: every 8- and 16-bit pattern (and edge values plus random ones of
    the wider types) as the sum, for every P up to 64, against the oracle's C division."""
    import torch
    np_dt = oracle.NP_CARRIER[dtype]
    es = oracle.dtype_size(dtype)
    if es <= 2:
        x = np.arange(1 << (8 * es), dtype=np.uint32).astype(np.uint8 if es == 1 else np.uint16).view(np_dt)
    else:
        x = oracle.fill(20000, dtype, "fullrange" if dtype in INT_DTYPES else "uniform_pm1", 77)
        if dtype in INT_DTYPES:
            info = np.iinfo(np_dt)
            edge = [info.min, info.min + 1, info.max, info.max - 1, 0, 1, 2, 63, 64, 65, 127, 128, 129]
            edge += [-1, -2, -63, -64, -65] if info.min < 0 else []
            x[:len(edge)] = np.array(edge, dtype=np_dt)
        else:
            tiny = np.finfo(np_dt).tiny
            x[:6] = np.array([0.0, -0.0, tiny, -tiny * 0.5, np.inf, np.nan], dtype=np_dt)
            x[6:100] *= tiny  # subnormal quotients
    zero = np.zeros_like(x)
    d_x, d_zero = to_dev(x), to_dev(zero)
    out = dev_empty(x.size, x.dtype)
    for P in list(range(1, 18)) + [24, 31, 32, 33, 48, 63, 64]:
        ins = [d_x] + [d_zero] * (P - 1)
        al.combine([out], ins, "avg", order="rank_asc", dtype=dtype, count=x.size)
        torch.cuda.synchronize()
        want = oracle.combine([x] + [zero] * (P - 1), dtype, "avg", "rank_asc")
        assert_bits_equal(to_host(out, x.dtype), want, dtype, "avg %s P=%d" % (dtype, P))


def test_avg_in_every_collective(al):
    """avg through reduce_scatter, reduce_scatterv (in place too), the combine into several buffers
    and the tree orders."""
    import torch
    P, n = 5, 7001
    for dtype in ("f32", "bf16", "i16", "u64"):
        ins = make_inputs(P, P * n, dtype, "avg")
        np_dt = ins[0].dtype
        want = oracle.reduce_scatter(ins, dtype, "avg", "pairwise_desc")
        recvs = [dev_empty(n, np_dt) for _ in range(P)]
        al.reduce_scatter(recvs, [to_dev(a) for a in ins], "avg", order="pairwise_desc", dtype=dtype, count=n)
        torch.cuda.synchronize()
        for b in range(P):
            assert_bits_equal(to_host(recvs[b], np_dt), want[b], dtype, "reduce_scatter avg %s block %d" % (dtype, b))
        bufs = [to_dev(a) for a in ins]
        al.reduce_scatter(bufs, bufs, "avg", order="pairwise_desc", dtype=dtype, count=n)
        torch.cuda.synchronize()
        for b in range(P):
            assert_bits_equal(to_host(bufs[b], np_dt)[:n], want[b], dtype, "in-place reduce_scatter avg %s" % dtype)
        counts = [n + 3, 0, 2 * n, 17, P * n - (n + 3) - 2 * n - 17]
        wantv = oracle.reduce_scatterv(ins, counts, dtype, "avg", "tree_halv")
        recvs = [dev_empty(max(c, 1), np_dt) for c in counts]
        al.reduce_scatterv(recvs, [to_dev(a) for a in ins], counts, "avg", order="tree_halv", dtype=dtype)
        torch.cuda.synchronize()
        for b in range(P):
            assert_bits_equal(to_host(recvs[b], np_dt)[:counts[b]], wantv[b], dtype, "reduce_scatterv avg %s" % dtype)
        for order in ("tree_dbl", "tree_binomial", "ring"):
            wanta = oracle.combine(ins, dtype, "avg", order, 2 if order == "ring" else 0)
            outs = run_combine(al, ins, dtype, "avg", order, 2 if order == "ring" else 0, nout=P)
            for o in outs:
                assert_bits_equal(o, wanta, dtype, "avg %s %s to %d buffers" % (dtype, order, P))


def test_errors(al):
    import torch
    a = [to_dev(np.zeros(16, np.float32)) for _ in range(2)]
    out = [dev_empty(16, np.float32)]
    with pytest.raises(al.AlError, match="Reduction operator not supported"):
        al.combine(out, a, 11)  # one past avg
    with pytest.raises(al.AlError, match="Reduction operator not supported"):
        al.combine(out, a, "band")
    with pytest.raises(al.AlError, match="Invalid algorithm"):
        al.combine(out, a, "sum", order=17)
    big = to_dev(np.zeros(40, np.float32))
    with pytest.raises(al.AlError) as e:
        al.combine([big[4:20]], [big[0:16], big[20:36]], "sum", dtype="f32", count=16)
    assert e.value.code == 5
    with pytest.raises(al.AlError):
        al.combine(out, [a[0]] * 65, "sum")
    # a pointer that is not aligned to its element type is refused (no kernel is launched)
    raw = to_dev(np.zeros(80, np.uint8))
    with pytest.raises(al.AlError, match="not aligned to its element type"):
        al.combine(out, [a[0], raw[1:65]], "sum", dtype="f32", count=16)
    with pytest.raises(al.AlError, match="not aligned to its element type"):
        al.reduce_scatter([raw[2:10], raw[40:48]], [a[0], a[1]], "sum", dtype="f32", count=2)
    with pytest.raises(al.AlError, match="not aligned to its element type"):
        al.ring_allreduce([a[0], raw[1:65]], "sum", dtype="f32", count=16)
    # zero-length is a no-op
    al.combine(out, a, "sum", count=0)
    torch.cuda.synchronize()


def test_combine_in_a_hip_graph(al):
    """The library only launches kernels, so a call can be captured into a HIP
    graph; every replay must give the eager result (fresh inputs each time)."""
    import torch
    P, n = 8, 300007
    ins = [to_dev(a) for a in make_inputs(P, n, "f32", "sum")]
    out = dev_empty(n, np.float32)
    al.combine([out], ins, "sum", order="tree_dbl")  # eager warm-up outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        al.combine([out], ins, "sum", order="tree_dbl")
    for rep in range(3):
        fresh = make_inputs(P, n, "f32", "sum", seed=500 + 10 * rep)
        for t, a in zip(ins, fresh):
            t.copy_(torch.from_numpy(a))       # eager work between the replays
        out.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = oracle.combine(fresh, "f32", "sum", "tree_dbl")
        assert_bits_equal(to_host(out, np.float32), want, "f32", "graph replay %d" % rep)


def test_collectives_in_a_hip_graph(al):
    """An allreduce to every rank (fold + spread), a Reduce_scatterv (ragged segments), an Allgatherv
    (spread for the large slice, the table-driven kernel for the small ones) and a fused ring captured
    into one graph; every replay, with fresh inputs, gives what the oracle gives."""
    import torch
    P, n = 4, (1 << 22) + 36  # 16 MiB and a bit: the combine takes its two steps, the ring its pieces
    counts = [300000, 0, 5, n - 300005]
    displs = [0, 300000, 300000, 300005]
    ins = [dev_empty(n, np.float32) for _ in range(P)]
    all_out = [dev_empty(n, np.float32) for _ in range(P)]
    rs_out = [dev_empty(max(c, 1), np.float32) for c in counts]
    ag_out = [dev_empty(n, np.float32) for _ in range(P)]
    ring = [dev_empty(n, np.float32) for _ in range(P)]

    def run():
        al.combine(all_out, ins, "sum", order="tree_dbl")
        al.reduce_scatterv(rs_out, ins, counts, "sum", order="pairwise_desc")
        al.allgatherv(ag_out, rs_out, counts, displs)
        for r in range(P):
            al.copy(ring[r], ins[r])
        al.ring_allreduce(ring, "sum", mode="fused")

    fresh = make_inputs(P, n, "f32", "sum", seed=900)
    for t, a in zip(ins, fresh):
        t.copy_(torch.from_numpy(a))
    run()  # eager warm-up outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        run()
    for rep in range(3):
        fresh = make_inputs(P, n, "f32", "sum", seed=910 + 10 * rep)
        for t, a in zip(ins, fresh):
            t.copy_(torch.from_numpy(a))
        for t in all_out + ag_out + ring:
            t.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want_all = oracle.combine(fresh, "f32", "sum", "tree_dbl")
        want_rs = oracle.reduce_scatterv(fresh, counts, "f32", "sum", "pairwise_desc")
        want_ag = np.concatenate([want_rs[q][:counts[q]] for q in range(P)])
        want_ring = oracle.ring_allreduce(fresh, "f32", "sum", (4 << 20) // 4)[0]
        for r in range(P):
            assert_bits_equal(to_host(all_out[r], np.float32), want_all, "f32", "replay %d allreduce rank %d" % (rep, r))
            assert_bits_equal(to_host(rs_out[r], np.float32)[:counts[r]], want_rs[r][:counts[r]], "f32",
                              "replay %d reduce_scatterv rank %d" % (rep, r))
            assert_bits_equal(to_host(ag_out[r], np.float32), want_ag, "f32", "replay %d allgatherv rank %d" % (rep, r))
            assert_bits_equal(to_host(ring[r], np.float32), want_ring, "f32", "replay %d ring rank %d" % (rep, r))


def test_reduce_scatterv_chained_wait_that_gives_up_is_reported(al):
    """The waits inside a chained in-place launch are bounded.  With the test's setting under which every
    wait that the tiling calls for gives up without looking at its flag (nothing is wrong with the device,
    every kernel ends normally, and the outcome does not depend on how fast anything runs) the result of
    the call is not valid: the query says so once, and a Reduce_scatterv that follows an unreported expiry
    refuses with ALAMD_ERR_TIMEOUT, after which everything works again."""
    import torch
    P, counts = 4, [1, 6_000_000, 3, 0]
    sends = make_inputs(P, sum(counts), "f32", "sum")
    want = oracle.reduce_scatterv(sends, counts, "f32", "sum", "rank_asc")
    assert not al.reduce_scatterv_wait_expired()
    try:
        al.set_chain_poll_limit(al.CHAIN_POLLS_NONE)
        bufs = [to_dev(a) for a in sends]
        al.reduce_scatterv(bufs, bufs, counts, "sum", order="rank_asc", dtype="f32")
        torch.cuda.synchronize()
        assert al.reduce_scatterv_wait_expired(), "no wait gave up although none was allowed a poll"
        assert not al.reduce_scatterv_wait_expired(), "reported once only"
        bufs = [to_dev(a) for a in sends]
        al.reduce_scatterv(bufs, bufs, counts, "sum", order="rank_asc", dtype="f32")  # expires again, not queried
        torch.cuda.synchronize()
    finally:
        al.set_chain_poll_limit(0)
    bufs = [to_dev(a) for a in sends]
    with pytest.raises(al.AlError, match="gave up waiting") as e:  # the next call reports it instead of running
        al.reduce_scatterv(bufs, bufs, counts, "sum", order="rank_asc", dtype="f32")
    assert e.value.code == 7
    al.reduce_scatterv(bufs, bufs, counts, "sum", order="rank_asc", dtype="f32")
    torch.cuda.synchronize()
    assert not al.reduce_scatterv_wait_expired()
    for b in range(P):
        assert_bits_equal(to_host(bufs[b], np.float32)[:counts[b]], want[b], "f32", "after the report, rank %d" % b)


def test_reduce_scatterv_captured_without_a_warm_up(al):
    """An in-place Reduce_scatterv whose block overlaps its own input, captured into a HIP graph on a stream
    that has never run one: the library may not allocate under capture, so without a reservation the call
    is refused with a message that names the remedy, and with alamd_reserve_scratch made beforehand the
    capture succeeds cold and every replay gives the oracle's bits."""
    import torch
    P, counts = 3, [1, 2_000_003, 7]
    total = sum(counts)
    src = [dev_empty(total, np.float32) for _ in range(P)]
    work = [dev_empty(total, np.float32) for _ in range(P)]

    def run():
        for r in range(P):
            al.copy(work[r], src[r])
        al.reduce_scatterv(work, work, counts, "sum", order="pairwise_desc", dtype="f32")

    cold = torch.cuda.Stream()
    with pytest.raises(al.AlError, match="alamd_reserve_scratch") as e:
        g0 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g0, stream=cold):
            run()
    assert e.value.code == 1
    torch.cuda.synchronize()
    del g0

    s = torch.cuda.Stream()
    al.reserve_scratch(counts[1] * 4, stream=s.cuda_stream)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        run()  # first ever call on this stream: nothing allocated, nothing synchronised
    for rep in range(3):
        fresh = [oracle.fill(total, "f32", "uniform_pm1", 900 + 10 * rep + r) for r in range(P)]
        for t, a in zip(src, fresh):
            t.copy_(torch.from_numpy(a))  # eager work between the replays
        for t in work:
            t.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = oracle.reduce_scatterv(fresh, counts, "f32", "sum", "pairwise_desc")
        for b in range(P):
            got = to_host(work[b], np.float32)
            assert_bits_equal(got[:counts[b]], want[b], "f32", "graph replay %d rank %d" % (rep, b))
            assert got[counts[b]:].tobytes() == fresh[b][counts[b]:].tobytes(), "bytes behind the result changed"
    del g
    al.release_scratch(stream=s.cuda_stream)
    al.release_scratch(stream=s.cuda_stream)  # nothing left to free: still fine


SETTINGS = [
    {},  # the defaults
    {"launch_bytes": 1 << 20, "two_step_min_total_bytes": 4096, "two_step_piece_bytes": 64 << 10,
     "ring_piece_bytes": 128 << 10, "spread_launch_bytes": 1 << 20, "spread_hbm_chunk_tiles": 8,
     "spread_hbm_launch_chunks": 1, "spread_cache_chunk_tiles": 8, "spread_cache_launch_chunks": 1},
    {"launch_bytes": 1 << 40, "two_step_min_outputs": 99, "spread_hbm_chunk_tiles": 24, "spread_hbm_launch_chunks": 3,
     "spread_launch_bytes": 1 << 40, "ring_piece_bytes": 1 << 40},
    {"two_step_min_total_bytes": 1, "two_step_min_outputs": 2, "two_step_piece_bytes": 1 << 20,
     "spread_cache_chunk_tiles": 16, "spread_cache_launch_chunks": 2, "launch_bytes": 3 << 20},
    # the streaming kernels: few waves per CU and three streams up front for every rank count, ...
    {"stream_wgs_per_cu": 4, "fold_front3_ranks": 2},
    # ... as many as fit and two up front for every rank count
    {"stream_wgs_per_cu": 32, "fold_front3_ranks": 1000, "launch_bytes": 1 << 22},
    # every fold / tree launch in the block shape, ...
    {"block_shape_from_bytes": 1, "block_shape_below_bytes": 1 << 60},
    # ... in many launches, ...
    {"block_shape_from_bytes": 1, "block_shape_below_bytes": 1 << 60, "launch_bytes": 1 << 20},
    # ... and none
    {"block_shape_below_bytes": 1},
]


@pytest.mark.parametrize("k", range(len(SETTINGS)))
def test_results_do_not_depend_on_the_launch_planners_sizes(al, k):
    """The sizes the launch planners cut their work by (bytes per launch, the thresholds and pieces of
    the two-step calls, the spread's chunks, the waves per CU and streams requested up front of the
    streaming kernels, the sizes between which a launch takes the block shape) only decide how the same work is spread over launches and waves:
    extreme settings give the bits of the defaults, i.e. the oracle's."""
    import torch
    P, n = 5, 1_300_007
    ins_h = make_inputs(P, n, "f32", "sum")
    try:
        for name, value in SETTINGS[k].items():
            al.tune(name, value)
            assert al.tuned(name) == value
        ins = [to_dev(a) for a in ins_h]
        outs = [dev_empty(n, np.float32) for _ in range(P)]
        al.combine(outs, ins, "sum", order="tree_dbl")
        one = dev_empty(n, np.float32)
        al.combine([one], ins, "sum", order="rank_asc")
        counts = [n // P + (1 if q < n % P else 0) for q in range(P)]
        displs = [sum(counts[:q]) for q in range(P)]
        rs = [dev_empty(c, np.float32) for c in counts]
        al.reduce_scatterv(rs, ins, counts, "sum", order="pairwise_desc")
        ag = [dev_empty(n, np.float32) for _ in range(P)]
        al.allgatherv(ag, rs, counts, displs)
        ring = [to_dev(a) for a in ins_h]
        al.ring_allreduce(ring, "sum", mode="fused")
        torch.cuda.synchronize()
    finally:
        for name in SETTINGS[k]:
            al.tune(name, 0)
    want_tree = oracle.combine(ins_h, "f32", "sum", "tree_dbl")
    want_fold = oracle.combine(ins_h, "f32", "sum", "rank_asc")
    want_rs = oracle.reduce_scatterv(ins_h, counts, "f32", "sum", "pairwise_desc")
    want_ring = oracle.ring_allreduce(ins_h, "f32", "sum", (4 << 20) // 4)[0]
    assert_bits_equal(to_host(one, np.float32), want_fold, "f32", "fold, settings %d" % k)
    for r in range(P):
        assert_bits_equal(to_host(outs[r], np.float32), want_tree, "f32", "allreduce rank %d, settings %d" % (r, k))
        assert_bits_equal(to_host(rs[r], np.float32), want_rs[r], "f32", "reduce_scatterv rank %d, settings %d" % (r, k))
        assert_bits_equal(to_host(ag[r], np.float32), np.concatenate(want_rs), "f32", "allgatherv rank %d, settings %d" % (r, k))
        assert_bits_equal(to_host(ring[r], np.float32), want_ring, "f32", "fused ring rank %d, settings %d" % (r, k))
    with pytest.raises(al.AlError):
        al.tune("no_such_size", 1)


@pytest.mark.parametrize("seed", range(6))
def test_reduce_scatterv_in_place_random_counts(al, seed):
    """In place, with random counts (zeros, a few elements, thousands), some ranks in place and some
    not: blocks that do not read what another writes share a launch, the others follow in order, the
    ones that overlap their own input are chained.  Every result against the oracle, and the bytes
    behind each result unchanged."""
    import torch
    rng = np.random.default_rng(1234 + seed)
    for _ in range(5):
        P = int(rng.choice([2, 3, 5, 8, 13, 33, 64]))
        kind = rng.integers(0, 3)
        if kind == 0:
            counts = [int(c) for c in rng.integers(0, 3000, P)]
        elif kind == 1:
            counts = [int(rng.choice([0, 1, 7, 500, 20000])) for _ in range(P)]
        else:  # ascending, so that late blocks are longer than early displacements
            counts = sorted(int(c) for c in rng.integers(1, 30000, P))
        if sum(counts) == 0:
            counts[0] = 5
        dtype, op = [("f32", "sum"), ("i32", "bxor"), ("bf16", "max")][int(rng.integers(0, 3))]
        order = ["rank_asc", "pairwise_desc", "tree_halv"][int(rng.integers(0, 3))]
        sends = make_inputs(P, sum(counts), dtype, op, seed=int(rng.integers(1, 1 << 20)))
        want = oracle.reduce_scatterv(sends, counts, dtype, op, order)
        bufs = [to_dev(a) for a in sends]
        in_place = [bool(rng.integers(0, 4)) for _ in range(P)]
        recvs = [bufs[b] if in_place[b] else dev_empty(max(counts[b], 1), sends[0].dtype) for b in range(P)]
        al.reduce_scatterv(recvs, bufs, counts, op, order=order, dtype=dtype)
        torch.cuda.synchronize()
        for b in range(P):
            got = to_host(recvs[b], sends[0].dtype)
            assert_bits_equal(got[:counts[b]], want[b], dtype, "P=%d counts %s... %s %s %s rank %d" % (
                P, counts[:6], dtype, op, order, b))
            if in_place[b]:
                assert got[counts[b]:].tobytes() == sends[b][counts[b]:].tobytes(), "rank %d: bytes behind the result changed" % b
