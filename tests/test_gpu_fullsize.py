"""Parity at the full sizes of the benchmark configurations (P = 8; 2^26 fp32, 2^27 bf16,
2^28 integers, a 516^3 fp64 grid).

Inputs are generated on the device by alamd_fill; the oracle regenerates the
same streams on the host tile by tile (the generator is counter-based), so
nothing but the result crosses PCIe.  Bit-exact."""
import numpy as np
import pytest

import oracle
from util import assert_bits_equal, to_dev

pytestmark = pytest.mark.gpu
P = 8


def device_inputs(al, torch, dtype, count, dist, seed):
    carrier = al.torch_dtype(dtype)
    ins = [torch.empty(count, dtype=carrier, device="cuda") for _ in range(P)]
    for r in range(P):
        al.fill(ins[r], dist, seed + r, dtype=dtype)
    return ins


@pytest.mark.parametrize("op,dist,order", [("sum", "uniform_pm1", "rank_asc"), ("prod", "uniform_09_11", "rank_asc"),
                                           ("sum", "uniform_pm1", "tree_dbl")])
def test_c2_fp32_full_size(al, op, dist, order):
    """C2: P=8 fp32 buffers of 2^26 elements, seed 1000+rank."""
    import torch
    n = 1 << 26
    ins = device_inputs(al, torch, "f32", n, dist, 1000)
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    al.combine([out], ins, op, order=order)
    torch.cuda.synchronize()
    want = oracle.combine_generated(P, n, "f32", op, order, 0, dist, 1000)
    assert_bits_equal(out.cpu().numpy(), want, "f32", "C2 %s %s" % (op, order))


def test_c2_bf16_full_size(al):
    import torch
    n = 1 << 27
    ins = device_inputs(al, torch, "bf16", n, "normal", 2000)
    out = torch.empty(n, dtype=torch.int16, device="cuda")
    al.combine([out], ins, "sum", order="rank_asc", dtype="bf16")
    torch.cuda.synchronize()
    want = oracle.combine_generated(P, n, "bf16", "sum", "rank_asc", 0, "normal", 2000)
    assert_bits_equal(out.cpu().numpy().view(np.uint16), want, "bf16", "C2 bf16")


@pytest.mark.parametrize("dtype,dist,seed", [("f32", "uniform_pm1", 1000), ("bf16", "normal", 2000), ("f64", "uniform_pm1", 1000),
                                             ("i32", "fullrange", 3000)])
def test_middling_sizes_in_the_block_shape(al, dtype, dist, seed):
    """Calls that move between 32 and 384 MiB in all and whose tiles of 16 KiB deal out evenly over the CUs
    run in such tiles with every load issued up front, by the library's own choice: 4 Mi elements per rank
    (buffers one element into their allocations, so with leading elements and a ragged last tile), one
    output and eight, fold and tree orders, float min under the order whose operand roles change from
    block to block; and the sizes either side of the two thresholds."""
    import torch
    assert al.tuned("block_shape_from_bytes") == 32 << 20 and al.tuned("block_shape_below_bytes") == 384 << 20
    es = al.dtype_size(dtype)
    carrier = al.torch_dtype(dtype)
    np_dt = oracle.NP_CARRIER[dtype]
    n = 1 << 22
    raw = [torch.empty(n + 1, dtype=carrier, device="cuda") for _ in range(P)]
    ins = [t[1:] for t in raw]
    for r in range(P):
        al.fill(ins[r], dist, seed + r, dtype=dtype)
    host = [t.cpu().numpy().view(np_dt) for t in ins]
    is_float = dtype in ("f32", "bf16", "f64")
    cases = [("sum", "rank_asc", 1), ("sum", "rank_asc", 8)]
    if is_float:
        cases += [("sum", "tree_rsg", 1), ("min", "tree_rsg", 2), ("sum", "tree_dbl", 8)]
    else:
        cases += [("max", "pairwise_desc", 2)]
    for op, order, nout in cases:
        want = oracle.combine(host, dtype, op, order)
        outs = [torch.empty(n + 1, dtype=carrier, device="cuda")[1:] for _ in range(nout)]
        al.combine(outs, ins, op, order=order, dtype=dtype)
        torch.cuda.synchronize()
        for o in outs:
            assert_bits_equal(o.cpu().numpy().view(np_dt), want, dtype, "%s %s %s to %d buffers" % (dtype, op, order, nout))
    # one tile of 16 KiB either side of where the shape changes (totals of 32 MiB and 384 MiB)
    for total in (32 << 20, 384 << 20):
        for delta in (-4096 // es, 0, 4096 // es):
            m = total // (P + 1) // es + delta
            if m > n:
                sub = [torch.empty(m, dtype=carrier, device="cuda") for _ in range(P)]
                for r in range(P):
                    al.fill(sub[r], dist, seed + r, dtype=dtype)
            else:
                sub = [t[:m] for t in ins]
            out = torch.empty(m, dtype=carrier, device="cuda")
            al.combine([out], sub, "sum", order="rank_asc", dtype=dtype)
            torch.cuda.synchronize()
            want = oracle.combine([t.cpu().numpy().view(np_dt) for t in sub], dtype, "sum", "rank_asc")
            assert_bits_equal(out.cpu().numpy().view(np_dt), want, dtype, "%s, %d elements per rank" % (dtype, m))
            del out, sub


@pytest.mark.parametrize("mode", ("stepwise", "fused"))
def test_c3_ring_full_size(al, mode):
    """C3: P=8 bf16 buffers of 2^27 elements, seed 2000+rank, 4 MiB chunks."""
    import torch
    n = 1 << 27
    bufs = device_inputs(al, torch, "bf16", n, "normal", 2000)
    al.ring_allreduce(bufs, "sum", chunk_bytes=4 << 20, mode=mode, dtype="bf16")
    torch.cuda.synchronize()
    for r in range(1, P):  # every logical rank ends with the same bytes
        assert torch.equal(bufs[0], bufs[r]), "rank %d differs from rank 0" % r
    got = bufs[0].cpu().numpy().view(np.uint16)
    for s in range(P):  # segment s is the ring-order fold that starts at rank s
        off, ln = oracle.ring_segment(n, P, s)
        want = oracle.combine_generated(P, ln, "bf16", "sum", "ring", s, "normal", 2000, off)
        assert_bits_equal(got[off:off + ln], want, "bf16", "C3 %s segment %d" % (mode, s))


@pytest.mark.parametrize("dtype", ("i32", "i64"))
def test_c4_integer_full_size(al, dtype):
    """C4: P=8 buffers of 2^28 full-range integers, seed 3000+rank; min / max / band / bor / bxor."""
    import torch
    n = 1 << 28
    ins = device_inputs(al, torch, dtype, n, "fullrange", 3000)
    out = torch.empty(n, dtype=al.torch_dtype(dtype), device="cuda")
    for op in ("min", "max", "band", "bor", "bxor"):
        al.combine([out], ins, op, dtype=dtype)
        torch.cuda.synchronize()
        want = oracle.combine_generated(P, n, dtype, op, "rank_asc", 0, "fullrange", 3000)
        got = out.cpu().numpy()
        assert got.tobytes() == want.tobytes(), "C4 %s %s" % (dtype, op)
        del want, got


def test_c4_uint8_logical_full_size(al):
    import torch
    n = 1 << 28
    ins = device_inputs(al, torch, "u8", n, "bool01", 3000)
    out = torch.empty(n, dtype=torch.uint8, device="cuda")
    for op in ("land", "lor", "lxor"):
        al.combine([out], ins, op, dtype="u8")
        torch.cuda.synchronize()
        want = oracle.combine_generated(P, n, "u8", op, "rank_asc", 0, "bool01", 3000)
        assert out.cpu().numpy().tobytes() == want.tobytes(), "C4 u8 %s" % op
    # a checksum of checksums: folding the halves separately gives the halves of the whole fold
    half = n // 2
    out2 = torch.empty(n, dtype=torch.uint8, device="cuda")
    al.combine([out2[:half]], [t[:half] for t in ins], "lxor", dtype="u8", count=half)
    al.combine([out2[half:]], [t[half:] for t in ins], "lxor", dtype="u8", count=half)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


def test_c5_halo_full_size(al):
    """C5: fp64, interior 512^3, halo 2, uniform[0,1) seed 4000; identity loopback."""
    import torch
    n, h = 512, 2
    side = n + 2 * h
    dims = (n, n, n)
    grid = torch.empty(side ** 3, dtype=torch.float64, device="cuda")
    al.fill(grid, "uniform_01", 4000)
    before = grid.clone()
    bufs = {f: torch.empty(al.halo_face_elems(dims, h, f), dtype=torch.float64, device="cuda") for f in range(6)}
    al.halo_pack(bufs, grid, dims, h)
    al.halo_unpack(grid, bufs, dims, h)
    torch.cuda.synchronize()
    host = oracle.fill(side ** 3, "f64", "uniform_01", 4000)
    assert before.cpu().numpy().tobytes() == host.tobytes()
    for f in range(6):
        assert bufs[f].cpu().numpy().tobytes() == oracle.halo_pack(host, n, n, n, h, f).tobytes(), "face %d" % f
    want = host
    for f in range(6):
        want = oracle.halo_unpack(want, oracle.halo_pack(host, n, n, n, h, f), n, n, n, h, f)
    got = grid.cpu().numpy()
    assert got.tobytes() == want.tobytes()
    # the interior is untouched and each ghost slab equals the matching interior slab
    g3, b3 = got.reshape(side, side, side), host.reshape(side, side, side)
    assert (g3[h:-h, h:-h, h:-h] == b3[h:-h, h:-h, h:-h]).all()
    assert (g3[h:-h, h:-h, :h] == b3[h:-h, h:-h, h:2 * h]).all()
    assert (g3[:h, h:-h, h:-h] == b3[h:2 * h, h:-h, h:-h]).all()


@pytest.mark.parametrize("P,cut", [(2, 16384), (8, 4096), (12, 2048)])
def test_multi_launch_boundaries(al, P, cut):
    """Counts around the launch cut (a power of two of 16 KiB tiles that depends on the number of
    ranks) and a ragged tail."""
    import torch
    tile = 16384 // 4
    for n in (cut * tile - 1, cut * tile + 1, 2 * cut * tile + 4099):
        ins = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(P)]
        for r in range(P):
            al.fill(ins[r], "uniform_pm1", 77 + r)
        out = torch.empty(n, dtype=torch.float32, device="cuda")
        al.combine([out], ins, "sum")
        torch.cuda.synchronize()
        want = oracle.combine_generated(P, n, "f32", "sum", "rank_asc", 0, "uniform_pm1", 77)
        assert_bits_equal(out.cpu().numpy(), want, "f32", "n=%d" % n)
        del ins, out


def test_buffers_beyond_4_gib(al):
    """Byte offsets past 2^32: two buffers of 4 GiB + 8 MiB + 4099 bytes, bitwise xor, checked in slices."""
    import torch
    n = (1 << 32) + (1 << 23) + 4099
    ins = [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(2)]
    for r in range(2):
        al.fill(ins[r], "fullrange", 900 + r, dtype="u8")
    out = torch.empty(n, dtype=torch.uint8, device="cuda")
    al.combine([out], ins, "bxor", dtype="u8")
    torch.cuda.synchronize()
    m = 1 << 22
    for lo in (0, (1 << 31) - m // 2, (1 << 32) - m // 2, n - m):
        want = oracle.combine_generated(2, m, "u8", "bxor", "rank_asc", 0, "fullrange", 900, lo)
        assert out[lo:lo + m].cpu().numpy().tobytes() == want.tobytes(), "slice at %d" % lo
    # a whole-buffer property: folding the result with one input again gives back the other input
    back = torch.empty(n, dtype=torch.uint8, device="cuda")
    al.combine([back], [out, ins[1]], "bxor", dtype="u8")
    torch.cuda.synchronize()
    assert torch.equal(back, ins[0])


def test_allgather_large_slices(al):
    """Slices of a few MB (below the 16 MiB from which a slice gets launches of its own); also in place."""
    import torch
    P = 5
    for count in (700001, 700004):  # 2.8 MB fp32 slices: byte path, then 16-byte aligned vector path
        sends = [torch.empty(count, dtype=torch.float32, device="cuda") for _ in range(P)]
        for r in range(P):
            al.fill(sends[r], "uniform_pm1", 60 + r)
        recvs = [torch.zeros(P * count, dtype=torch.float32, device="cuda") for _ in range(P)]
        al.allgather(recvs, sends, count=count)
        torch.cuda.synchronize()
        want = torch.cat(sends)
        for r in range(P):
            assert torch.equal(recvs[r], want), "rank %d" % r
        host = np.concatenate([oracle.fill(count, "f32", "uniform_pm1", 60 + r) for r in range(P)])
        assert recvs[0].cpu().numpy().tobytes() == host.tobytes()
    # a 16-byte-aligned in-place form: slices of 700004 elements
    count = 700004
    bufs = [torch.zeros(P * count, dtype=torch.float32, device="cuda") for _ in range(P)]
    views = [bufs[r][r * count:(r + 1) * count] for r in range(P)]
    for r in range(P):
        al.fill(views[r], "uniform_pm1", 80 + r, count=count)
    want = torch.cat([v.clone() for v in views])
    al.allgather(bufs, views, count=count)
    torch.cuda.synchronize()
    for r in range(P):
        assert torch.equal(bufs[r], want), "in place, rank %d" % r
    # bytes: sources and receive buffers at odd addresses, slice length not a multiple of 16
    count = (1 << 20) + 3
    raw = [torch.empty(count + 8, dtype=torch.uint8, device="cuda") for _ in range(P)]
    sends = [raw[r][1 + r % 3:1 + r % 3 + count] for r in range(P)]
    for r in range(P):
        al.fill(sends[r], "fullrange", 90 + r, dtype="u8", count=count)
    rraw = [torch.full((P * count + 8,), 0xEE, dtype=torch.uint8, device="cuda") for _ in range(P)]
    recvs = [rraw[r][3:3 + P * count] for r in range(P)]
    al.allgather(recvs, sends, dtype="u8", count=count)
    torch.cuda.synchronize()
    want = torch.cat(sends)
    for r in range(P):
        assert torch.equal(recvs[r], want), "bytes, rank %d" % r
        assert bool((rraw[r][:3] == 0xEE).all()) and bool((rraw[r][3 + P * count:] == 0xEE).all())


@pytest.mark.parametrize("order", ("rank_asc", "tree_dbl"))
@pytest.mark.parametrize("inplace", (False, True))
def test_large_combine_to_several_outputs(al, order, inplace):
    """From 16 MiB up a result for several outputs is folded into the first and then spread: one
    count below that and three around 64 MiB, three ranks, separate and in-place outputs."""
    import torch
    P = 3
    piece = (64 << 20) // 4
    for n in (300000, piece - 4, piece + 4, piece + (1 << 20) + 12):
        ins = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(P)]
        for r in range(P):
            al.fill(ins[r], "uniform_pm1", 500 + r)
        outs = ins if inplace else [torch.zeros(n, dtype=torch.float32, device="cuda") for _ in range(P)]
        al.combine(outs, ins, "sum", order=order)
        torch.cuda.synchronize()
        want = oracle.combine_generated(P, n, "f32", "sum", order, 0, "uniform_pm1", 500)
        for j in range(P):
            assert_bits_equal(outs[j].cpu().numpy(), want, "f32", "n=%d output %d" % (n, j))


def test_allgatherv_large_slices_with_tails(al):
    """Slices of 1 to 2 MB whose byte counts are not multiples of 16, placed back to front."""
    import torch
    P = 4
    counts = [300001, 0, 262147, 500003]
    # slots 16-byte aligned, with gaps, laid out from the last rank to the first
    displs, at = [0] * P, 4
    for q in reversed(range(P)):
        displs[q] = at
        at += (counts[q] + 3) // 4 * 4 + 8
    extent = max(d + c for d, c in zip(displs, counts))
    sends = [torch.empty(max(c, 1), dtype=torch.float32, device="cuda") for c in counts]
    for r in range(P):
        al.fill(sends[r], "uniform_pm1", 700 + r)
    recvs = [torch.full((extent,), -3.0, dtype=torch.float32, device="cuda") for _ in range(P)]
    al.allgatherv(recvs, sends, counts, displs)
    torch.cuda.synchronize()
    want = np.full(extent, -3.0, dtype=np.float32)
    for q in range(P):
        want[displs[q]:displs[q] + counts[q]] = oracle.fill(max(counts[q], 1), "f32", "uniform_pm1", 700 + q)[:counts[q]]
    for r in range(P):
        assert recvs[r].cpu().numpy().tobytes() == want.tobytes(), "rank %d" % r


@pytest.mark.parametrize("P,count", [(3, 3 * 300000), (8, 8 * 262144 + 8 * 4)])
def test_fused_ring_large_segments(al, P, count):
    """Segments above 1 MiB, one fold launch; same bits as the stepwise ring."""
    import torch
    bufs = [torch.empty(count, dtype=torch.float32, device="cuda") for _ in range(P)]
    for r in range(P):
        al.fill(bufs[r], "uniform_pm1", 800 + r)
    step = [b.clone() for b in bufs]
    al.ring_allreduce(bufs, "sum", mode="fused")
    al.ring_allreduce(step, "sum", mode="stepwise")
    torch.cuda.synchronize()
    host = [oracle.fill(count, "f32", "uniform_pm1", 800 + r) for r in range(P)]
    want = oracle.ring_allreduce(host, "f32", "sum", (4 << 20) // 4)[0]
    for r in range(P):
        assert_bits_equal(bufs[r].cpu().numpy(), want, "f32", "fused rank %d" % r)
        assert torch.equal(step[r], bufs[r])


@pytest.mark.parametrize("op", ("sum", "prod", "min", "max"))
@pytest.mark.parametrize("dtype", ("bf16", "f16"))
def test_every_pair_of_16bit_patterns(al, dtype, op):
    """One combine step over all 2^32 (inout, in) pairs of 16-bit patterns: NaNs, infinities,
    subnormals, signed zeros, ties and every rounding case, against the oracle's
    widen / one fp32 operation / narrow (src/mpi_impl.cpp:61-145)."""
    import torch
    rows = 1 << 10
    n = rows << 16
    allbits = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    b_host = np.tile(allbits, rows)
    b_dev = torch.from_numpy(b_host.view(np.int16)).cuda()
    a_dev = torch.empty(n, dtype=torch.int16, device="cuda")
    out = torch.empty(n, dtype=torch.int16, device="cuda")
    idx = torch.arange(n, dtype=torch.int32, device="cuda") >> 16
    nan_above = 0x7f80 if dtype == "bf16" else 0x7c00
    for base in range(0, 1 << 16, rows):
        a_host = np.repeat(allbits[base:base + rows], 1 << 16)
        v = idx + base
        a_dev.copy_(torch.where(v >= (1 << 15), v - (1 << 16), v).to(torch.int16))
        al.combine([out], [a_dev, b_dev], op, order="rank_asc", dtype=dtype)
        want = torch.from_numpy(oracle.step(a_host, b_host, dtype, op).view(np.int16)).cuda()
        both_nan = ((out & 0x7fff) > nan_above) & ((want & 0x7fff) > nan_above)
        if not bool(((out == want) | both_nan).all()):
            assert_bits_equal(out.cpu().numpy().view(np.uint16), want.cpu().numpy().view(np.uint16), dtype,
                              "%s %s, inout patterns from %#x" % (dtype, op, base))


@pytest.mark.parametrize("dtype,op", [("u16", o) for o in ("sum", "prod", "min", "max", "lor", "land", "lxor", "bor",
                                                            "band", "bxor")] + [("i16", "min"), ("i16", "max"),
                                                                                ("i16", "prod")])
def test_every_pair_of_16bit_integers(al, dtype, op):
    """All 2^32 operand pairs; sum, prod and the bit/logical operators do not depend on the
    sign, so the signed type adds only min, max (and prod once more, for the wrap)."""
    import torch
    rows = 1 << 10
    n = rows << 16
    allbits = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    npdt = oracle.NP_CARRIER[dtype]
    b_host = np.tile(allbits, rows).view(npdt)
    b_dev = torch.from_numpy(b_host.view(np.int16)).cuda()
    a_dev = torch.empty(n, dtype=torch.int16, device="cuda")
    out = torch.empty(n, dtype=torch.int16, device="cuda")
    idx = torch.arange(n, dtype=torch.int32, device="cuda") >> 16
    for base in range(0, 1 << 16, rows):
        a_host = np.repeat(allbits[base:base + rows], 1 << 16).view(npdt)
        v = idx + base
        a_dev.copy_(torch.where(v >= (1 << 15), v - (1 << 16), v).to(torch.int16))
        al.combine([out], [a_dev, b_dev], op, order="rank_asc", dtype=dtype)
        want = torch.from_numpy(oracle.step(a_host, b_host, dtype, op).view(np.int16)).cuda()
        if not bool((out == want).all()):
            assert_bits_equal(out.cpu().numpy().view(npdt), want.cpu().numpy().view(npdt), dtype,
                              "%s %s, first operands from %#x" % (dtype, op, base))


@pytest.mark.parametrize("dtype", ("u8", "i8"))
def test_every_pair_of_bytes_in_every_lane(al, dtype):
    """All 65536 byte pairs under all ten operators, each pair visiting all 16 byte
    positions of a 128-bit vector, plus a ragged tail for the element path."""
    import torch
    npdt = oracle.NP_CARRIER[dtype]
    n = 65536 * 16 + 11
    j = np.arange(n, dtype=np.int64)
    j = j + j // 65536
    a = (j % 256).astype(np.uint8).view(npdt)
    b = ((j // 256) % 256).astype(np.uint8).view(npdt)
    a_dev, b_dev = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    out = torch.empty(n, dtype=a_dev.dtype, device="cuda")
    for op in ("sum", "prod", "min", "max", "lor", "land", "lxor", "bor", "band", "bxor"):
        al.combine([out], [a_dev, b_dev], op, order="rank_asc", dtype=dtype)
        torch.cuda.synchronize()
        assert_bits_equal(out.cpu().numpy().view(npdt), oracle.step(a, b, dtype, op), dtype, "%s %s" % (dtype, op))


def test_allgather_slices_over_several_launches(al):
    """Slices longer than one spread launch covers (32 MiB of a source), byte counts that are not
    multiples of 16, sources and receive buffers at odd addresses; separate buffers and in place."""
    import torch
    P = 3
    count = (40 << 20) + 5
    raw = [torch.empty(count + 8, dtype=torch.uint8, device="cuda") for _ in range(P)]
    sends = [raw[r][1 + r:1 + r + count] for r in range(P)]
    for r in range(P):
        al.fill(sends[r], "fullrange", 170 + r, dtype="u8", count=count)
    rraw = [torch.full((P * count + 8,), 0xEE, dtype=torch.uint8, device="cuda") for _ in range(P)]
    recvs = [rraw[r][3:3 + P * count] for r in range(P)]
    al.allgather(recvs, sends, dtype="u8", count=count)
    torch.cuda.synchronize()
    want = torch.cat(sends)
    for q in range(P):
        host = oracle.fill(count, "u8", "fullrange", 170 + q)
        assert want[q * count:(q + 1) * count].cpu().numpy().tobytes() == host.tobytes()
    for r in range(P):
        assert torch.equal(recvs[r], want), "rank %d" % r
        assert bool((rraw[r][:3] == 0xEE).all()) and bool((rraw[r][3 + P * count:] == 0xEE).all())
    # in place: rank r's slice already sits at r * count of its own buffer
    bufs = [torch.full((P * count,), 0x11, dtype=torch.uint8, device="cuda") for _ in range(P)]
    for r in range(P):
        bufs[r][r * count:(r + 1) * count].copy_(sends[r])
    al.allgather(bufs, [bufs[r][r * count:(r + 1) * count] for r in range(P)], dtype="u8", count=count)
    torch.cuda.synchronize()
    for r in range(P):
        assert torch.equal(bufs[r], want), "in place, rank %d" % r


@pytest.mark.parametrize("order", ("rank_asc", "tree_halv"))
def test_reduce_scatter_more_than_eight_large_segments(al, order):
    """Twelve blocks of 6 MB: more segments than one launch takes side by side, each longer than
    one launch's share of tiles, with a ragged tail."""
    import torch
    P = 12
    count = 1500000 + 3
    sends = [oracle.fill(P * count, "f32", "uniform_pm1", 900 + r) for r in range(P)]
    d_sends = [to_dev(s) for s in sends]
    recvs = [torch.zeros(count, dtype=torch.float32, device="cuda") for _ in range(P)]
    al.reduce_scatter(recvs, d_sends, "sum", order=order, count=count)
    torch.cuda.synchronize()
    want = oracle.reduce_scatter(sends, "f32", "sum", order)
    for r in range(P):
        assert_bits_equal(recvs[r].cpu().numpy(), want[r], "f32", "%s rank %d" % (order, r))


@pytest.mark.parametrize("inplace", (False, True))
def test_combine_to_several_outputs_in_pieces(al, inplace):
    """A result above 256 MiB for three outputs alternates fold and spread over 128 MiB pieces:
    300 MiB + 5 elements, every output equal to the one-output result, windows against the oracle."""
    import torch
    P = 3
    n = (300 << 20) // 4 + 5
    ins = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(P)]
    for r in range(P):
        al.fill(ins[r], "uniform_pm1", 1500 + r)
    single = torch.empty(n, dtype=torch.float32, device="cuda")
    al.combine([single], ins, "sum", order="tree_dbl")
    outs = ins if inplace else [torch.zeros(n, dtype=torch.float32, device="cuda") for _ in range(P)]
    al.combine(outs, ins, "sum", order="tree_dbl")
    torch.cuda.synchronize()
    for j in range(P):
        assert torch.equal(outs[j].view(torch.int32), single.view(torch.int32)), "output %d" % j
    m = 1 << 16
    piece = (128 << 20) // 4
    for lo in (0, piece - m // 2, 2 * piece - m // 2, n - m):
        want = oracle.combine_generated(P, m, "f32", "sum", "tree_dbl", 0, "uniform_pm1", 1500, lo)
        assert_bits_equal(single[lo:lo + m].cpu().numpy(), want, "f32", "window at %d" % lo)


@pytest.mark.parametrize("P,count", [(3, 3 * 6000000 + 2), (5, 5 * 4200000 + 3)])
def test_fused_ring_in_pieces(al, P, count):
    """Fused ring allreduce above 16 MiB: 64 MiB pieces over ragged segments; same bits as the oracle's
    chunk-by-chunk ring and as the stepwise mode."""
    import torch
    bufs = [torch.empty(count, dtype=torch.float32, device="cuda") for _ in range(P)]
    for r in range(P):
        al.fill(bufs[r], "uniform_pm1", 1600 + r)
    step = [b.clone() for b in bufs]
    al.ring_allreduce(bufs, "sum", mode="fused")
    al.ring_allreduce(step, "sum", mode="stepwise")
    torch.cuda.synchronize()
    host = [oracle.fill(count, "f32", "uniform_pm1", 1600 + r) for r in range(P)]
    want = oracle.ring_allreduce(host, "f32", "sum", (4 << 20) // 4)[0]
    for r in range(P):
        assert_bits_equal(bufs[r].cpu().numpy(), want, "f32", "fused rank %d" % r)
        assert torch.equal(step[r].view(torch.int32), bufs[r].view(torch.int32))


@pytest.mark.parametrize("order", ("rank_asc", "tree_halv"))
def test_reduce_scatterv_very_unequal_blocks(al, order):
    """One block of 144 MB beside blocks of 20 bytes, nothing and 36 MB: the long blocks get launches of
    their own (several each), the short ones theirs."""
    import torch
    P = 4
    counts = [36000000, 5, 0, 9000001]
    total = sum(counts)
    sends = [oracle.fill(total, "f32", "uniform_pm1", 1700 + r) for r in range(P)]
    d_sends = [to_dev(s) for s in sends]
    recvs = [torch.zeros(max(c, 1), dtype=torch.float32, device="cuda") for c in counts]
    al.reduce_scatterv(recvs, d_sends, counts, "sum", order=order)
    torch.cuda.synchronize()
    want = oracle.reduce_scatterv(sends, counts, "f32", "sum", order)
    for b in range(P):
        assert_bits_equal(recvs[b].cpu().numpy()[:counts[b]], want[b], "f32", "%s block %d" % (order, b))


@pytest.mark.parametrize("P", (24, 64))
def test_many_ranks_medium_sizes(al, P):
    """Sixty-four (and twenty-four) ranks at sizes where the launch planner puts many short segments side by
    side and the allgather groups several short slices per launch: allgather of odd-sized byte slices,
    Reduce_scatter, fused and stepwise ring allreduce, combine into every rank's buffer."""
    import torch
    # allgather: slices of about 300 KB, byte counts not multiples of 16
    count = 300007
    sends = [oracle.fill(count, "u8", "fullrange", 2100 + r) for r in range(P)]
    recvs = [torch.full((P * count,), 0xEE, dtype=torch.uint8, device="cuda") for _ in range(P)]
    al.allgather(recvs, [to_dev(s) for s in sends], dtype="u8", count=count)
    torch.cuda.synchronize()
    want = np.concatenate(sends)
    for r in (0, P // 2, P - 1):
        assert recvs[r].cpu().numpy().tobytes() == want.tobytes(), "allgather rank %d" % r
    del recvs
    # reduce_scatter: blocks of about 600 KB
    blk = 150001
    host = [oracle.fill(P * blk, "i32", "fullrange", 2200 + r) for r in range(P)]
    d_sends = [to_dev(h) for h in host]
    outs = [torch.zeros(blk, dtype=torch.int32, device="cuda") for _ in range(P)]
    al.reduce_scatter(outs, d_sends, "sum", dtype="i32", count=blk)
    torch.cuda.synchronize()
    want_rs = oracle.reduce_scatter(host, "i32", "sum", "rank_asc")
    for r in range(P):
        assert_bits_equal(outs[r].cpu().numpy().view(np.int32), want_rs[r], "i32", "reduce_scatter rank %d" % r)
    # ring allreduce over the same buffers (in place), fused against stepwise against the oracle
    n = P * blk
    step = [d.clone() for d in d_sends]
    al.ring_allreduce(d_sends, "sum", mode="fused", dtype="i32")
    al.ring_allreduce(step, "sum", mode="stepwise", dtype="i32")
    torch.cuda.synchronize()
    want_ar = oracle.combine(host, "i32", "sum", "rank_asc")
    for r in (0, 1, P - 1):
        assert_bits_equal(d_sends[r].cpu().numpy().view(np.int32), want_ar, "i32", "fused ring rank %d" % r)
        assert torch.equal(step[r], d_sends[r])
    # combine of float inputs into every rank's buffer (two steps: fold, then spread to P - 1 buffers)
    m = 4200011
    fin = [oracle.fill(m, "f32", "uniform_pm1", 2300 + r) for r in range(P)]
    d_in = [to_dev(f) for f in fin]
    al.combine(d_in, d_in, "sum", order="rank_asc")
    torch.cuda.synchronize()
    want_c = oracle.combine(fin, "f32", "sum", "rank_asc")
    for r in (0, P - 1):
        assert_bits_equal(d_in[r].cpu().numpy(), want_c, "f32", "combine rank %d" % r)


@pytest.mark.parametrize("order", ("rank_asc", "tree_dbl"))
def test_reduce_scatterv_blocks_taken_longest_first(al, order):
    """Sixteen blocks that alternate between about 10 MB and a few KB: in rank order every launch would
    hold one long block, so the launches take the blocks sorted by length; every block still lands in
    its own rank's buffer, folded from its own starting rank."""
    import torch
    P = 16
    counts = [2600000 + 4099 * r if r % 2 == 0 else 700 + r for r in range(P)]
    counts[5] = 0
    total = sum(counts)
    sends = [oracle.fill(total, "f32", "uniform_pm1", 2500 + r) for r in range(P)]
    d_sends = [to_dev(s) for s in sends]
    recvs = [torch.zeros(max(c, 1), dtype=torch.float32, device="cuda") for c in counts]
    al.reduce_scatterv(recvs, d_sends, counts, "sum", order=order)
    torch.cuda.synchronize()
    want = oracle.reduce_scatterv(sends, counts, "f32", "sum", order)
    for b in range(P):
        assert_bits_equal(recvs[b].cpu().numpy()[:counts[b]], want[b], "f32", "%s block %d" % (order, b))
