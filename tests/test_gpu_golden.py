"""The HIP library against the MPICH golden vectors in tests/golden, through the C ABI and with
no oracle in between: what MPI_Allreduce / MPI_Reduce / MPI_Reduce_scatter_block / MPI_Reduce_scatter of
MPICH 3.3.2 returned for these inputs (the calls the reference's MPI backend forwards to,
include/aluminum/mpi/allreduce.hpp:38-44, mpi/reduce.hpp:41-49, mpi/reduce_scatter.hpp:40-46), and what
their non-blocking forms returned where that differs (the calls its host-transfer backend makes,
include/aluminum/ht/allreduce.hpp:76-79, ht/reduce.hpp:72-82), is what the GPU must return, bit for bit,
under the order that alamd_reference_order names for that call, root, type and message size, for 2 to 64
ranks - including the cases with NaNs, zeros of both signs and infinities planted in
every operand position, where the bits depend on which operand of every pair is the inoutvec."""
import glob
import gzip
import json
import os

import numpy as np
import pytest

import oracle
from util import assert_bits_equal, dev_empty, mpich_order, planted_specials, to_dev, to_host

pytestmark = pytest.mark.gpu

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "mpich_P*.json.gz")),
                key=lambda p: int(os.path.basename(p)[7:-8]))
IDS = [os.path.basename(p)[:-8] for p in GOLDEN]
COLL = {"allreduce": 0, "reduce": 1, "reduce_scatter": 2, "reduce_scatterv": 2}


def load(path):
    with gzip.open(path, "rt") as f:
        return json.load(f)


def arr(hexstr, dtype):
    return np.frombuffer(bytes.fromhex(hexstr), dtype=oracle.NP_CARRIER[dtype]).copy()


def inputs_of(c, P, n):
    if "in" in c:
        return [arr(h, c["dtype"]) for h in c["in"]]
    if c["note"] == "specials":
        return [planted_specials(n, c["dtype"], r) for r in range(P)]
    return [oracle.fill(n, c["dtype"], c["dist"], c["seed_base"] + r) for r in range(P)]


def lean(P):
    """From 32 ranks on a fixture holds a small set of cases and one output for an allreduce."""
    return P >= 32


def library_order(al, coll, P, count, dtype, root=0, blocking=False):
    """What the library itself picks for the non-blocking MPI call (which the host-transfer backend makes) or
    the blocking one; the tests also hold it against the table in util.mpich_order."""
    order, start = al.reference_order(coll + ("_blocking" if blocking else ""), P, count, dtype, root)
    want = mpich_order(coll, dtype, count if coll in ("allreduce", "reduce") else 0, P, root, total=count,
                       blocking=blocking)
    assert (order, start) == want, (coll, P, count, dtype, root, order, start, want)
    return order, start


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_allreduce_vectors_on_the_gpu(al, path):
    import torch
    doc = load(path)
    P, seen = doc["P"], 0
    for c in doc["cases"]:
        if c["coll"] != "allreduce":
            continue
        dt, op, n = c["dtype"], c["op"], c["n"]
        ins = inputs_of(c, P, n)
        d_ins = [to_dev(a) for a in ins]
        for blocking in (True, False):  # MPI_Allreduce, MPI_Iallreduce
            want = arr(c["out"][0] if blocking else c.get("out_nonblocking", c["out"][0]), dt)
            order, start = library_order(al, "allreduce", P, n, dt, blocking=blocking)
            outs = [dev_empty(n, ins[0].dtype) for _ in range(P)]
            al.combine(outs, d_ins, op, order=order, start=start, dtype=dt, count=n)
            torch.cuda.synchronize()
            what = "P=%d %s %s n=%d %s (%s)" % (P, dt, op, n, c["note"], order)
            for r in range(P):
                assert_bits_equal(to_host(outs[r], ins[0].dtype), want, dt, what + " rank %d" % r)
        seen += 1
    assert seen >= (7 if lean(P) else 18)


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_reduce_vectors_on_the_gpu(al, path):
    """MPI_Reduce to the first, second and last rank."""
    import torch
    doc = load(path)
    P, seen, roots = doc["P"], 0, set()
    for c in doc["cases"]:
        if c["coll"] != "reduce":
            continue
        dt, op, n, root = c["dtype"], c["op"], c["n"], c["root"]
        npdt = oracle.NP_CARRIER[dt]
        d_ins = [to_dev(a) for a in inputs_of(c, P, n)]
        for blocking in (True, False):  # MPI_Reduce, MPI_Ireduce
            order, start = library_order(al, "reduce", P, n, dt, root, blocking=blocking)
            out = dev_empty(n, npdt)
            al.combine([out], d_ins, op, order=order, start=start, dtype=dt, count=n)
            torch.cuda.synchronize()
            got = to_host(out, npdt)
            what = "P=%d %s %s n=%d root %d %s (%s)" % (P, dt, op, n, root, c["note"], order)
            if "out" in c:
                assert_bits_equal(got, arr(c["out"] if blocking else c.get("out_nonblocking", c["out"]), dt), dt, what)
            else:
                assert c["nonblocking_in_place_same"]
                assert "%016x" % oracle.checksum(got) == c["out_checksum"], what
                assert_bits_equal(got[:8], arr(c["out_head"], dt), dt, what)
        seen += 1
        roots.add(root)
    assert seen >= (12 if lean(P) else 30) and roots == {0, 1, P - 1}


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_reduce_scatter_vectors_on_the_gpu(al, path):
    import torch
    doc = load(path)
    P, seen = doc["P"], 0
    for c in doc["cases"]:
        if c["coll"] != "reduce_scatter":
            continue
        dt, op, count = c["dtype"], c["op"], c["n"]
        npdt = oracle.NP_CARRIER[dt]
        order, _ = library_order(al, "reduce_scatter", P, P * count, dt)
        ins = inputs_of(c, P, P * count)
        d_sends = [to_dev(a) for a in ins]
        d_recvs = [dev_empty(count, npdt) for _ in range(P)]
        al.reduce_scatter(d_recvs, d_sends, op, order=order, dtype=dt, count=count)
        torch.cuda.synchronize()
        for r in range(P):
            got = to_host(d_recvs[r], npdt)
            if "out" in c:
                assert_bits_equal(got, arr(c["out"][r], dt), dt, "reduce_scatter short P=%d %s rank %d" % (P, dt, r))
            else:
                assert "%016x" % oracle.checksum(got) == c["out_checksum"][r], (P, dt, r)
                assert_bits_equal(got[:8], arr(c["out_head"][r], dt), dt, "head")
        seen += 1
    assert seen >= (3 if lean(P) else 8)


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_reduce_scatterv_vectors_on_the_gpu(al, path):
    """MPI_Reduce_scatter with uneven counts, below and above 512 KiB in all."""
    import torch
    doc = load(path)
    P = doc["P"]
    cases = [c for c in doc["cases"] if c["coll"] == "reduce_scatterv"]
    assert len(cases) == (0 if lean(P) else 8)
    for c in cases:
        dt, counts, total = c["dtype"], c["counts"], c["n"]
        npdt = oracle.NP_CARRIER[dt]
        order, _ = library_order(al, "reduce_scatter", P, total, dt)
        d_sends = [to_dev(a) for a in inputs_of(c, P, total)]
        d_recvs = [dev_empty(max(k, 1), npdt) for k in counts]
        al.reduce_scatterv(d_recvs, d_sends, counts, c["op"], order=order, dtype=dt)
        torch.cuda.synchronize()
        for b in range(P):
            got = to_host(d_recvs[b], npdt)[:counts[b]]
            what = "reduce_scatterv P=%d %s rank %d (%s)" % (P, dt, b, order)
            if "out" in c:
                assert_bits_equal(got, arr(c["out"][b], dt)[:counts[b]], dt, what)
            else:
                assert "%016x" % oracle.checksum(got) == c["out_checksum"][b], what
                if counts[b]:
                    assert_bits_equal(got[:8], arr(c["out_head"][b], dt), dt, what)


MPIEXEC = "/opt/conda/bin/mpiexec"
MPI_PROGRAM = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "mpi_baseline")


@pytest.mark.skipif(not (os.path.exists(MPIEXEC) and os.path.exists(MPI_PROGRAM)),
                    reason="needs mpiexec and the built oracle/mpi_baseline")
@pytest.mark.parametrize("P", (2, 3, 4, 5, 8))
def test_live_mpi_allreduce_and_reduce_against_the_gpu(al, P):
    """MPI_Allreduce and MPI_Reduce (MPI_SUM, MPI_FLOAT) run now, on this machine's host cores, over
    generated inputs (uniform[-1,1), seed 1000+rank), against the GPU's combine of the same inputs under
    the order the library names: equal checksums."""
    import subprocess
    import torch
    for n in (300, 513, (1 << 16) + 1, 1 << 20):
        for root in (-1, 0, P - 1):  # -1: allreduce
            p = subprocess.run([MPIEXEC, "-n", str(P), MPI_PROGRAM, str(n), "0", "1", str(root)], capture_output=True,
                               text=True, timeout=120)
            line = [l for l in p.stdout.splitlines() if l.startswith("{")]
            assert p.returncode == 0 and line, (p.stdout, p.stderr)
            want = json.loads(line[-1])["checksum"]
            ins = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(P)]
            out = torch.empty(n, dtype=torch.float32, device="cuda")
            for r in range(P):
                al.fill(ins[r], "uniform_pm1", 1000 + r)
            order, start = library_order(al, "allreduce" if root < 0 else "reduce", P, n, "f32", max(root, 0))
            al.combine([out], ins, "sum", order=order, start=start)
            torch.cuda.synchronize()
            assert "%016x" % oracle.checksum(out.cpu().numpy()) == want, "P=%d n=%d root=%d" % (P, n, root)
