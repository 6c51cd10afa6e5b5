"""GPU parity of the ring emulation, the halo faces, the stream flags and the
test-support entry points, through the C ABI, against the CPU oracle."""
import threading
import time

import numpy as np
import pytest

import oracle
from util import FLOAT_DTYPES, assert_bits_equal, dev_empty, to_dev, to_host

pytestmark = pytest.mark.gpu


def ring_inputs(P, n, dtype, op):
    dist = {"sum": "normal", "prod": "uniform_09_11", "min": "uniform_pm1", "max": "uniform_pm1",
            "bxor": "fullrange", "lor": "bool01", "avg": "normal"}[op]
    if dtype not in FLOAT_DTYPES and op in ("sum", "prod", "min", "max", "avg"):
        dist = "fullrange"
    return [oracle.fill(n, dtype, dist, 2000 + r) for r in range(P)]


@pytest.mark.parametrize("dtype,op", [("bf16", "sum"), ("f32", "sum"), ("f16", "prod"), ("f64", "max"),
                                      ("bf16", "min"), ("i32", "sum"), ("u8", "lor"), ("u64", "bxor"),
                                      ("bf16", "avg"), ("f32", "avg"), ("i8", "avg"), ("i64", "avg")])
@pytest.mark.parametrize("mode", ("stepwise", "fused"))
def test_ring_allreduce(al, dtype, op, mode):
    import torch
    es = oracle.dtype_size(dtype)
    for P in (1, 2, 3, 8):
        for n in (P * 64, P * 4096 + 3, 5, 10000):
            for chunk_elems in (1, 7, 512):
                if n > 1000 and chunk_elems == 1:
                    continue
                bufs = ring_inputs(P, n, dtype, op)
                want = oracle.ring_allreduce(bufs, dtype, op, chunk_elems)
                d = [to_dev(b) for b in bufs]
                al.ring_allreduce(d, op, chunk_bytes=chunk_elems * es, mode=mode, dtype=dtype, count=n)
                torch.cuda.synchronize()
                for r in range(P):
                    assert_bits_equal(to_host(d[r], bufs[0].dtype), want[r], dtype,
                                      "ring %s %s %s P=%d n=%d chunk=%d rank %d" % (mode, dtype, op, P, n, chunk_elems, r))


@pytest.mark.parametrize("dtype,op", [("bf16", "sum"), ("f32", "prod"), ("i16", "min")])
def test_ring_reduce_scatter_then_allgather(al, dtype, op):
    import torch
    es = oracle.dtype_size(dtype)
    P, n = 8, 8 * 2048
    bufs = ring_inputs(P, n, dtype, op)
    want_rs = oracle.ring_reduce_scatter(bufs, dtype, op, 300)
    d = [to_dev(b) for b in bufs]
    al.ring_reduce_scatter(d, op, chunk_bytes=300 * es, mode="stepwise", dtype=dtype, count=n)
    torch.cuda.synchronize()
    # the stepwise emulation reproduces every intermediate partial too
    for r in range(P):
        assert_bits_equal(to_host(d[r], bufs[0].dtype), want_rs[r], dtype, "stepwise reduce-scatter rank %d" % r)
    want_ag = oracle.ring_allgather(want_rs, dtype, 300)
    al.ring_allgather(d, chunk_bytes=300 * es, dtype=dtype, count=n)
    torch.cuda.synchronize()
    for r in range(P):
        assert_bits_equal(to_host(d[r], bufs[0].dtype), want_ag[r], dtype, "allgather rank %d" % r)
    # fused reduce-scatter: rank r owns segment (r+1) mod P afterwards
    d = [to_dev(b) for b in bufs]
    al.ring_reduce_scatter(d, op, chunk_bytes=300 * es, mode="fused", dtype=dtype, count=n)
    torch.cuda.synchronize()
    for r in range(P):
        off, ln = oracle.ring_segment(n, P, (r + 1) % P)
        assert_bits_equal(to_host(d[r], bufs[0].dtype)[off:off + ln], want_rs[r][off:off + ln], dtype,
                          "fused reduce-scatter rank %d" % r)


@pytest.mark.parametrize("dtype,op", [("bf16", "sum"), ("f32", "max"), ("u8", "bxor"), ("f64", "prod")])
@pytest.mark.parametrize("mode", ("stepwise", "fused"))
def test_ring_ragged_segments_and_offsets(al, dtype, op, mode):
    """Counts that are not multiples of P (segments differ by one element and start off 16-byte
    boundaries), buffers that are only element-aligned, several tiles per segment."""
    import torch
    for P, n in ((3, 3 * 20000 + 2), (8, 8 * 5000 + 5), (5, 4)):
        host = ring_inputs(P, n, dtype, op)
        want = oracle.ring_allreduce(host, dtype, op, 4096)
        pads = [np.zeros(1 + r % 2, host[0].dtype) for r in range(P)]
        bufs = [to_dev(np.concatenate([pads[r], host[r]]))[pads[r].size:] for r in range(P)]
        al.ring_allreduce(bufs, op, chunk_bytes=4096 * host[0].itemsize, mode=mode, dtype=dtype, count=n)
        torch.cuda.synchronize()
        for r in range(P):
            assert_bits_equal(to_host(bufs[r], host[0].dtype), want[r], dtype, "%s P=%d rank %d" % (mode, P, r))


@pytest.mark.parametrize("dtype,op", [("bf16", "sum"), ("f32", "prod"), ("i16", "min"), ("f64", "avg")])
@pytest.mark.parametrize("mode", ("stepwise", "fused"))
def test_ring_allreduce_from_separate_send_buffers(al, dtype, op, mode):
    """Al::Allreduce's form with a send and a receive buffer per rank: the same bits as in place, the
    send buffers untouched; also with some ranks in place and the others not, and at a size that
    takes the fused form's fold-then-spread path."""
    import torch
    es = oracle.dtype_size(dtype)
    for P, n in ((1, 10), (2, 4099), (5, 70_001), (8, (18 << 20) // es + 5)):
        bufs = ring_inputs(P, n, dtype, op)
        want = oracle.ring_allreduce(bufs, dtype, op, 512)
        for in_place in ([False] * P, [r % 2 == 0 for r in range(P)]):
            sends = [to_dev(b) for b in bufs]
            recvs = [sends[r] if in_place[r] else dev_empty(n, bufs[0].dtype) for r in range(P)]
            al.ring_allreduce(recvs, op, chunk_bytes=512 * es, mode=mode, dtype=dtype, count=n, sends=sends)
            torch.cuda.synchronize()
            for r in range(P):
                assert_bits_equal(to_host(recvs[r], bufs[0].dtype), want[r], dtype,
                                  "ring %s from send buffers, P=%d n=%d rank %d" % (mode, P, n, r))
                if not in_place[r]:
                    assert to_host(sends[r], bufs[0].dtype).tobytes() == bufs[r].tobytes(), "send buffer %d changed" % r
    # a receive buffer that overlaps another rank's send buffer is refused
    a = to_dev(oracle.fill(200, dtype, "fullrange" if dtype == "i16" else "uniform_pm1", 1))
    b = dev_empty(100, a.cpu().numpy().dtype if False else bufs[0].dtype)
    with pytest.raises(al.AlError) as e:
        al.ring_allreduce([a[:100], b], op, mode=mode, dtype=dtype, count=100, sends=[b, a[50:150]])
    assert e.value.code == 5


def test_ring_errors(al):
    bufs = [to_dev(np.zeros(64, np.float32)) for _ in range(4)]
    with pytest.raises(al.AlError):
        al.ring_allreduce(bufs, "sum", chunk_bytes=6)
    with pytest.raises(al.AlError):
        al.ring_allreduce(bufs, "sum", chunk_bytes=0)
    with pytest.raises(al.AlError, match="Reduction operator not supported"):
        al.ring_allreduce(bufs, "lor")  # a logical operator on a float type
    with pytest.raises(al.AlError):
        al.ring_allreduce([bufs[0], bufs[0]], "sum")


@pytest.mark.parametrize("np_dtype", (np.float64, np.float32, np.uint8, np.int16))
@pytest.mark.parametrize("dims,h", [((8, 6, 5), 2), ((16, 16, 16), 1), ((33, 7, 9), 3), ((4, 4, 4), 4),
                                    ((64, 48, 40), 2)])
def test_halo_pack_unpack(al, np_dtype, dims, h):
    import torch
    nx, ny, nz = dims
    rng = np.random.default_rng(4000)
    alloc = (nz + 2 * h, ny + 2 * h, nx + 2 * h)
    if np.issubdtype(np_dtype, np.floating):
        grid = rng.random(alloc).astype(np_dtype)
    else:
        grid = rng.integers(0, 120, alloc).astype(np_dtype)
    d_grid = to_dev(grid.reshape(-1))
    bufs = {f: dev_empty(oracle.halo_face_elems(nx, ny, nz, h, f), np_dtype) for f in range(6)}
    for f in range(6):
        assert al.halo_face_elems(dims, h, f) == oracle.halo_face_elems(nx, ny, nz, h, f)
    al.halo_pack(bufs, d_grid, dims, h)
    torch.cuda.synchronize()
    want_grid = grid.reshape(-1).copy()
    for f in range(6):
        want = oracle.halo_pack(grid.reshape(-1), nx, ny, nz, h, f)
        got = to_host(bufs[f], np_dtype)
        assert got.tobytes() == want.tobytes(), "pack face %d" % f
        want_grid = oracle.halo_unpack(want_grid, want, nx, ny, nz, h, f)
    # identity loopback: what was packed is what is received
    al.halo_unpack(d_grid, bufs, dims, h)
    torch.cuda.synchronize()
    assert to_host(d_grid, np_dtype).tobytes() == want_grid.tobytes(), "unpack"
    # a subset of faces in one call leaves the others alone
    d_grid2 = to_dev(grid.reshape(-1))
    al.halo_unpack(d_grid2, {1: bufs[1], 4: bufs[4]}, dims, h)
    torch.cuda.synchronize()
    w2 = oracle.halo_unpack(grid.reshape(-1), to_host(bufs[1], np_dtype), nx, ny, nz, h, 1)
    w2 = oracle.halo_unpack(w2, to_host(bufs[4], np_dtype), nx, ny, nz, h, 4)
    assert to_host(d_grid2, np_dtype).tobytes() == w2.tobytes(), "subset unpack"


def test_halo_pack_does_not_depend_on_the_load_policy(al):
    """The cache policy of the pack's grid loads is a measurement setting: every policy packs the same bytes."""
    import torch
    nx, ny, nz, h = 64, 40, 24, 2
    rng = np.random.default_rng(4100)
    grid = rng.random((nz + 2 * h, ny + 2 * h, nx + 2 * h))
    d_grid = to_dev(grid.reshape(-1))
    want = [oracle.halo_pack(grid.reshape(-1), nx, ny, nz, h, f) for f in range(6)]
    try:
        for policy in range(5):
            al.tune("halo_load_policy", policy)
            bufs = {f: dev_empty(oracle.halo_face_elems(nx, ny, nz, h, f), np.float64) for f in range(6)}
            al.halo_pack(bufs, d_grid, (nx, ny, nz), h)
            torch.cuda.synchronize()
            for f in range(6):
                assert to_host(bufs[f], np.float64).tobytes() == want[f].tobytes(), "policy %d face %d" % (policy, f)
    finally:
        al.tune("halo_load_policy", 0)


def test_halo_errors(al):
    grid = to_dev(np.zeros(6 * 6 * 6, np.float64))
    buf = {0: dev_empty(8, np.float64)}
    with pytest.raises(al.AlError):
        al.halo_pack(buf, grid, (2, 2, 2), 3)  # halo wider than the interior


@pytest.mark.parametrize("dtype", oracle.DTYPES)
def test_fill_matches_oracle(al, dtype):
    import torch
    n = 70001
    for dist in oracle.DISTS:
        t = dev_empty(n, oracle.NP_CARRIER[dtype])
        al.fill(t, dist, 4242, idx0=12345678901, dtype=dtype, count=n)
        torch.cuda.synchronize()
        want = oracle.fill(n, dtype, dist, 4242, 12345678901)
        assert_bits_equal(to_host(t, oracle.NP_CARRIER[dtype]), want, dtype, "fill %s %s" % (dtype, dist))


@pytest.mark.parametrize("dtype", ("bf16", "f16"))
def test_narrow_all_float32_patterns(al, dtype):
    """Every one of the 2^32 fp32 bit patterns narrows to the oracle's result."""
    import torch
    step = 1 << 27
    narrow = oracle.f32_to_bf16 if dtype == "bf16" else oracle.f32_to_f16
    src = torch.empty(step, dtype=torch.int32, device="cuda")
    dst = torch.empty(step, dtype=torch.int16, device="cuda")
    base = torch.arange(step, dtype=torch.int64, device="cuda")
    for k in range(0, 1 << 32, step):
        vals = base + k
        src.copy_(torch.where(vals >= (1 << 31), vals - (1 << 32), vals).to(torch.int32))
        al.narrow_f32(dst, src, dtype)
        torch.cuda.synchronize()
        host_src = (np.arange(k, k + step, dtype=np.uint64).astype(np.uint32)).view(np.float32)
        assert_bits_equal(to_host(dst, np.uint16), narrow(host_src), dtype, "narrow %s at %#x" % (dtype, k))


@pytest.mark.parametrize("dtype", ("bf16", "f16"))
def test_widen_all_16bit_patterns(al, dtype):
    import torch
    allbits = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    src = to_dev(allbits)
    dst = dev_empty(1 << 16, np.float32)
    al.widen_f32(dst, src, dtype)
    torch.cuda.synchronize()
    want = oracle.bf16_to_f32(allbits) if dtype == "bf16" else oracle.f16_to_f32(allbits)
    assert_bits_equal(to_host(dst, np.float32), want, "f32", "widen")


def test_copy(al):
    import torch
    for n in (0, 1, 15, 16, 4096, 100003):
        a = np.random.default_rng(n).integers(0, 255, n).astype(np.uint8)
        src, dst = to_dev(a) if n else dev_empty(0, np.uint8), dev_empty(n, np.uint8)
        al.copy(dst, src, nbytes=n)
        torch.cuda.synchronize()
        if n:
            assert to_host(dst, np.uint8).tobytes() == a.tobytes()
    # any byte alignment on either side; the bytes around the destination stay untouched
    n = 100003
    a = np.random.default_rng(7).integers(0, 255, n + 8).astype(np.uint8)
    src = to_dev(a)
    for so, do in ((1, 0), (0, 3), (5, 2)):
        dst = to_dev(np.full(n + 16, 0xEE, np.uint8))
        al.copy(dst[do:], src[so:], nbytes=n)
        torch.cuda.synchronize()
        got = to_host(dst, np.uint8)
        assert got[do:do + n].tobytes() == a[so:so + n].tobytes()
        assert (got[:do] == 0xEE).all() and (got[do + n:] == 0xEE).all()


# ---- stream flags ------------------------------------------------------------

def flag_modes(al):
    return ["kernel"] + (["memop"] if al.capi.memops_supported() else [])


def test_flag_initial_and_host_side(al):
    f = al.Flag(1)
    assert f.query() == 1  # created "complete", like GPUStatusFlag
    f.signal(0)
    assert f.query() == 0
    f.signal(7)
    assert f.query() == 7
    assert not f.timed_out()
    f.destroy()


def test_flag_write_orders_after_prior_work(al):
    """record(): the word flips only once the stream's earlier work is done."""
    import torch
    for mode in flag_modes(al):
        f = al.Flag(1)
        x = torch.zeros(1 << 24, device="cuda")
        torch.cuda.synchronize()
        f.signal(0)                      # host stores 0 ...
        for _ in range(20):
            x += 1.0
        f.write(1, mode=mode)            # ... the stream stores 1 when it gets there
        deadline = time.time() + 30
        while f.query() != 1 and time.time() < deadline:
            time.sleep(0.0005)
        assert f.query() == 1, mode
        torch.cuda.synchronize()
        assert float(x[0]) == 20.0 and float(x[-1]) == 20.0
        f.destroy()


def test_flag_wait_blocks_stream_until_signal(al):
    """wait(): work enqueued behind the wait does not start before the host signals."""
    import torch
    for mode in flag_modes(al):
        gate, done = al.Flag(0), al.Flag(0)
        s = torch.cuda.Stream()
        y = torch.zeros(1024, device="cuda")
        torch.cuda.synchronize()
        try:
            with torch.cuda.stream(s):
                # a bounded spin in kernel mode so the kernel ends even if the test dies
                gate.wait(1, mode=mode, max_spins=(1 << 22) if mode == "kernel" else 0)
                y += 1.0
                done.write(1, mode=mode)
            time.sleep(0.2)
            assert done.query() == 0, "stream ran past an unsignalled wait (%s)" % mode
        finally:
            gate.signal(1)
        s.synchronize()
        assert done.query() == 1
        assert float(y[0]) == 1.0
        assert not gate.timed_out()
        gate.destroy()
        done.destroy()


def test_flag_bounded_wait_gives_up(al):
    """A kernel wait with a spin limit ends by itself and says so."""
    import torch
    f = al.Flag(0)
    f.wait(1, mode="kernel", max_spins=200)
    torch.cuda.synchronize()
    assert f.timed_out()
    f.destroy()


def test_flag_signal_from_another_thread(al):
    """The progress-thread pattern: a host thread polls one flag and signals another."""
    import torch
    for mode in flag_modes(al):
        started, go = al.Flag(1), al.Flag(0)
        x = torch.zeros(16, device="cuda")
        torch.cuda.synchronize()

        def progress():
            deadline = time.time() + 30
            while started.query() != 1 and time.time() < deadline:
                time.sleep(0.0002)
            go.signal(1)

        started.signal(0)
        th = threading.Thread(target=progress)
        th.start()
        started.write(1, mode=mode)
        go.wait(1, mode=mode, max_spins=(1 << 22) if mode == "kernel" else 0)
        x += 2.0
        th.join()
        torch.cuda.synchronize()
        assert float(x[3]) == 2.0 and not go.timed_out()
        started.destroy()
        go.destroy()


def test_flag_pool_reuse(al):
    """Flags come from pooled pinned slabs: many create / destroy cycles are cheap and each flag
    starts with the value asked for, whatever its previous owner left."""
    t0 = time.time()
    flags = [al.Flag(k & 1) for k in range(300)]  # more than one slab
    for k, f in enumerate(flags):
        assert f.query() == (k & 1)
        f.signal(1234)
    for f in flags:
        f.destroy()
    for _ in range(2000):
        f = al.Flag(7)
        assert f.query() == 7 and not f.timed_out()
        f.destroy()
    assert time.time() - t0 < 20
