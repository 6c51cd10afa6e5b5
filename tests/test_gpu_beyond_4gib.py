"""Buffers, blocks and grids whose byte offsets pass 2^32, for every entry point besides the plain
fold (which tests/test_gpu_fullsize.py covers): allgather, reduce_scatter, the ring, in-place
reduce_scatterv (chained), copy, tree and descending orders, halo faces.

Inputs are generated on the device; whole buffers are compared on the device against torch's
element-wise operations (integer xor and wrapping add are exact there), and slices around 2^31
and 2^32 bytes against the CPU oracle, which regenerates the same streams.  Bit-exact."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

BIG = (1 << 32) + (1 << 23) + 4099  # bytes: 4 GiB + 8 MiB + 4099
SLICE = 1 << 22


def _check_slices(out, n, want_of, what):
    """Compares [lo, lo + SLICE) of a device byte buffer with what the oracle regenerates, at the
    start, around 2^31 and 2^32, and at the end."""
    for lo in (0, (1 << 31) - SLICE // 2, (1 << 32) - SLICE // 2, n - SLICE):
        if lo < 0 or lo + SLICE > n:
            continue
        assert out[lo:lo + SLICE].cpu().numpy().tobytes() == want_of(lo).tobytes(), "%s: slice at %d" % (what, lo)


def test_allgather_beyond_4_gib(al):
    """Receive buffers of 3 x 1.5 GiB: slices that start and end past 2^32 bytes; separate and in place."""
    import torch
    P = 3
    count = (3 << 29) + 4099 * 16 + 5  # bytes per slice, not a multiple of 16
    sends = [torch.empty(count, dtype=torch.uint8, device="cuda") for _ in range(P)]
    for r in range(P):
        al.fill(sends[r], "fullrange", 300 + r, dtype="u8")
    recvs = [torch.zeros(P * count, dtype=torch.uint8, device="cuda") for _ in range(P)]
    al.allgather(recvs, sends, dtype="u8", count=count)
    torch.cuda.synchronize()
    for r in range(P):
        for q in range(P):
            assert torch.equal(recvs[r][q * count:(q + 1) * count], sends[q]), "rank %d slice %d" % (r, q)
    # against the generator itself, where slice 2 crosses 2^32
    lo = (1 << 32) - 2 * count - SLICE // 2
    want = oracle.fill(SLICE, "u8", "fullrange", 302, lo)
    assert recvs[1][2 * count + lo:2 * count + lo + SLICE].cpu().numpy().tobytes() == want.tobytes()
    del sends
    # in place: every rank's slice already lies in its receive buffer
    for r in range(P):
        recvs[r].zero_()
        al.fill(recvs[r][r * count:(r + 1) * count], "fullrange", 310 + r, dtype="u8", count=count)
    keep = [recvs[r][r * count:(r + 1) * count].clone() for r in range(P)]
    al.allgather(recvs, [recvs[r][r * count:(r + 1) * count] for r in range(P)], dtype="u8", count=count)
    torch.cuda.synchronize()
    for r in range(P):
        for q in range(P):
            assert torch.equal(recvs[r][q * count:(q + 1) * count], keep[q]), "in place, rank %d slice %d" % (r, q)


@pytest.mark.parametrize("order", ("rank_asc", "tree_halv"))
def test_reduce_scatter_beyond_4_gib(al, order):
    """Two send buffers of 4 GiB + 8 MiB + 4100 bytes: the second rank's block ends past 2^32."""
    import torch
    P = 2
    count = (BIG + 1) // 2  # bytes per block
    n = P * count
    sends = [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(P)]
    for r in range(P):
        al.fill(sends[r], "fullrange", 400 + r, dtype="u8")
    recvs = [torch.zeros(count, dtype=torch.uint8, device="cuda") for _ in range(P)]
    al.reduce_scatter(recvs, sends, "bxor", order=order, dtype="u8", count=count)
    torch.cuda.synchronize()
    for r in range(P):
        assert torch.equal(recvs[r], torch.bitwise_xor(sends[0][r * count:(r + 1) * count],
                                                        sends[1][r * count:(r + 1) * count])), "rank %d" % r
    lo = count - SLICE  # the end of rank 1's block: offsets just below 2 * count in the send buffers
    want = oracle.combine_generated(2, SLICE, "u8", "bxor", "rank_asc", 0, "fullrange", 400, count + lo)
    assert recvs[1][lo:].cpu().numpy().tobytes() == want.tobytes()


@pytest.mark.parametrize("mode", ("stepwise", "fused"))
def test_ring_allreduce_beyond_4_gib(al, mode):
    """Two rank buffers of 2^30 + 2^21 + 5 int32 each (4 GiB + 8 MiB + 20 bytes): the second ring segment
    starts past 2^31 bytes and ends past 2^32."""
    import torch
    P = 2
    count = (1 << 30) + (1 << 21) + 5
    bufs = [torch.empty(count, dtype=torch.int32, device="cuda") for _ in range(P)]
    for r in range(P):
        al.fill(bufs[r], "fullrange", 500 + r, dtype="i32")
    want = bufs[0] + bufs[1]  # wraps like the step does
    al.ring_allreduce(bufs, "sum", mode=mode, dtype="i32", count=count)
    torch.cuda.synchronize()
    for r in range(P):
        assert torch.equal(bufs[r], want), "rank %d" % r
    m = SLICE // 4
    for lo in (0, (1 << 29) - m // 2, (1 << 30) - m // 2, count - m):
        ref = oracle.combine_generated(2, m, "i32", "sum", "rank_asc", 0, "fullrange", 500, lo)
        assert bufs[1][lo:lo + m].cpu().numpy().tobytes() == ref.tobytes(), "slice at element %d" % lo


def test_reduce_scatterv_in_place_beyond_4_gib(al):
    """In place with a short first block and a second block of more than 4 GiB: rank 1's result
    overlaps its own input, shifted by the first block's 70003 bytes, so its launch is chained."""
    import torch
    counts = [70003, BIG]
    n = sum(counts)
    bufs = [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(2)]
    for r in range(2):
        al.fill(bufs[r], "fullrange", 600 + r, dtype="u8")
    want1 = torch.bitwise_xor(bufs[0][counts[0]:], bufs[1][counts[0]:])
    want0 = torch.bitwise_xor(bufs[0][:counts[0]], bufs[1][:counts[0]])
    al.reduce_scatterv(bufs, bufs, counts, "bxor", dtype="u8")
    torch.cuda.synchronize()
    assert not al.reduce_scatterv_wait_expired()
    assert torch.equal(bufs[0][:counts[0]], want0)
    assert torch.equal(bufs[1][:counts[1]], want1)
    _check_slices(bufs[1], counts[1],
                  lambda lo: oracle.combine_generated(2, SLICE, "u8", "bxor", "rank_asc", 0, "fullrange", 600,
                                                      counts[0] + lo), "rank 1's block")


def test_copy_beyond_4_gib(al):
    import torch
    src = torch.empty(BIG + 3, dtype=torch.uint8, device="cuda")
    al.fill(src, "fullrange", 700, dtype="u8")
    dst = torch.zeros(BIG + 3, dtype=torch.uint8, device="cuda")
    al.copy(dst[3:], src[:BIG], nbytes=BIG)  # differently aligned
    torch.cuda.synchronize()
    assert torch.equal(dst[3:], src[:BIG]) and int(dst[:3].sum()) == 0


@pytest.mark.parametrize("order", ("tree_dbl", "pairwise_desc"))
def test_float_orders_beyond_4_gib(al, order):
    """Three fp32 buffers of 4 GiB + 8 MiB + 20 bytes under a tree order and a descending fold."""
    import torch
    P = 3
    count = (1 << 30) + (1 << 21) + 5
    ins = [torch.empty(count, dtype=torch.float32, device="cuda") for _ in range(P)]
    for r in range(P):
        al.fill(ins[r], "uniform_pm1", 800 + r)
    out = torch.empty(count, dtype=torch.float32, device="cuda")
    al.combine([out], ins, "sum", order=order)
    torch.cuda.synchronize()
    m = SLICE // 4
    for lo in (0, (1 << 29) - m // 2, (1 << 30) - m // 2, count - m):
        want = oracle.combine_generated(P, m, "f32", "sum", order, 0, "uniform_pm1", 800, lo)
        assert out[lo:lo + m].cpu().numpy().tobytes() == want.tobytes(), "slice at element %d" % lo


def test_halo_grid_beyond_4_gib(al):
    """A 1024 x 1024 x 524 fp64 allocation (4.1 GiB): plane and row offsets pass 2^32 bytes.  Pack, then
    unpack into the ghost slabs of the same sides; faces and ghost slabs against the slabs of a copy."""
    import torch
    h = 2
    dims = (1020, 1020, 520)  # x, y, z
    sx, sy, sz = (d + 2 * h for d in dims)
    grid = torch.empty(sx * sy * sz, dtype=torch.float64, device="cuda")
    al.fill(grid, "uniform_01", 4500)
    before = grid.clone().view(sz, sy, sx)
    bufs = {f: torch.empty(al.halo_face_elems(dims, h, f), dtype=torch.float64, device="cuda") for f in range(6)}
    al.halo_pack(bufs, grid, dims, h)
    al.halo_unpack(grid, bufs, dims, h)
    torch.cuda.synchronize()
    g3 = grid.view(sz, sy, sx)
    inner = (slice(h, -h), slice(h, -h), slice(h, -h))
    assert torch.equal(g3[inner], before[inner])
    # (interior slab the face holds, ghost slab it lands in): faces -x +x -y +y -z +z; axis 2 is x
    lo_in, hi_in, lo_gh, hi_gh = slice(h, 2 * h), slice(-2 * h, -h), slice(0, h), slice(-h, None)
    for f, (axis, src, dst) in enumerate([(2, lo_in, lo_gh), (2, hi_in, hi_gh), (1, lo_in, lo_gh), (1, hi_in, hi_gh),
                                          (0, lo_in, lo_gh), (0, hi_in, hi_gh)]):
        take, put = list(inner), list(inner)
        take[axis], put[axis] = src, dst
        slab = before[tuple(take)]
        assert torch.equal(bufs[f], slab.contiguous().view(-1)), "face %d" % f
        assert torch.equal(g3[tuple(put)], slab), "ghost slab of face %d" % f


def test_eight_buffers_of_16_gib(al):
    """Half of the 288 GB: eight 16 GiB inputs and one output, bitwise xor.  Slices against the oracle,
    and a whole-buffer property: folding the result with seven inputs again gives back the eighth."""
    import torch
    P, n = 8, (1 << 34) + 4099
    free, _ = torch.cuda.mem_get_info()
    if free < (P + 2) * n + (4 << 30):
        pytest.skip("needs %d GiB of free device memory" % (((P + 2) * n >> 30) + 4))
    ins = [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(P)]
    for r in range(P):
        al.fill(ins[r], "fullrange", 900 + r, dtype="u8")
    out = torch.empty(n, dtype=torch.uint8, device="cuda")
    al.combine([out], ins, "bxor", dtype="u8")
    torch.cuda.synchronize()
    for lo in (0, (1 << 32) - SLICE // 2, (1 << 33) + 12345, n - SLICE):
        want = oracle.combine_generated(P, SLICE, "u8", "bxor", "rank_asc", 0, "fullrange", 900, lo)
        assert out[lo:lo + SLICE].cpu().numpy().tobytes() == want.tobytes(), "slice at %d" % lo
    back = torch.empty(n, dtype=torch.uint8, device="cuda")
    al.combine([back], [out] + ins[1:], "bxor", dtype="u8")
    torch.cuda.synchronize()
    same = torch.equal(back, ins[0])
    del ins, out, back
    torch.cuda.empty_cache()  # give the 160 GiB back: other processes of the test run allocate too
    assert same
