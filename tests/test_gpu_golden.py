"""The HIP library against the MPICH golden vectors in tests/golden, through the C ABI and with
no oracle in between: what MPI_Allreduce / MPI_Reduce_scatter_block / MPI_Reduce_scatter of
MPICH 3.3.2 returned for these inputs (the calls the reference's MPI backend forwards to,
include/aluminum/mpi/allreduce.hpp:38-44, mpi/reduce_scatter.hpp:40-46) is what the GPU must
return, bit for bit, under the order the front end's `automatic` picks for that message size."""
import glob
import gzip
import json
import os

import numpy as np
import pytest

import oracle
from util import assert_bits_equal, dev_empty, to_dev, to_host

pytestmark = pytest.mark.gpu

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "mpich_P*.json.gz")))
IDS = [os.path.basename(p)[:-8] for p in GOLDEN]


def load(path):
    with gzip.open(path, "rt") as f:
        return json.load(f)


def arr(hexstr, dtype):
    return np.frombuffer(bytes.fromhex(hexstr), dtype=oracle.NP_CARRIER[dtype]).copy()


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_allreduce_vectors_on_the_gpu(al, path):
    import torch
    doc = load(path)
    P, seen = doc["P"], 0
    for c in doc["cases"]:
        if c["coll"] != "allreduce":
            continue
        dt, op, n = c["dtype"], c["op"], c["n"]
        ins = [arr(h, dt) for h in c["in"]]
        want = arr(c["out"][0], dt)
        # Al::Allreduce, automatic: binomial tree up to 2048 bytes, doubling tree above
        order = "tree_binomial" if n * ins[0].itemsize <= 2048 else "tree_dbl"
        d_ins = [to_dev(a) for a in ins]
        outs = [dev_empty(n, ins[0].dtype) for _ in range(P)]
        al.combine(outs, d_ins, op, order=order, dtype=dt, count=n)
        torch.cuda.synchronize()
        what = "P=%d %s %s n=%d %s" % (P, dt, op, n, c["note"])
        for r in range(P):
            assert_bits_equal(to_host(outs[r], ins[0].dtype), want, dt, what + " rank %d" % r)
        seen += 1
    assert seen >= 12


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
        if "in" in c:  # short message: recursive halving
            ins = [arr(h, dt) for h in c["in"]]
            order = "tree_halv"
        else:          # long message: pairwise exchange; inputs are the generator's, outputs kept as checksums
            ins = [oracle.fill(P * count, dt, c["dist"], c["seed_base"] + r) for r in range(P)]
            order = "pairwise_desc"
        d_sends = [to_dev(a) for a in ins]
        d_recvs = [dev_empty(count, npdt) for _ in range(P)]
        al.reduce_scatter(d_recvs, d_sends, op, order=order, dtype=dt, count=count)
        torch.cuda.synchronize()
        for r in range(P):
            got = to_host(d_recvs[r], npdt)
            if "in" in c:
                assert_bits_equal(got, arr(c["out"][r], dt), dt, "reduce_scatter short P=%d rank %d" % (P, r))
            else:
                assert "%016x" % oracle.checksum(got) == c["out_checksum"][r], (P, r)
                assert_bits_equal(got[:8], arr(c["out_head"][r], dt), dt, "head")
        seen += 1
    assert seen >= 4


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_reduce_scatterv_vectors_on_the_gpu(al, path):
    import torch
    doc = load(path)
    P = doc["P"]
    for c in [c for c in doc["cases"] if c["coll"] == "reduce_scatterv"]:
        dt, counts = c["dtype"], c["counts"]
        npdt = oracle.NP_CARRIER[dt]
        ins = [arr(h, dt) for h in c["in"]]
        d_sends = [to_dev(a) for a in ins]
        d_recvs = [dev_empty(max(k, 1), npdt) for k in counts]
        al.reduce_scatterv(d_recvs, d_sends, counts, c["op"], order="tree_halv", dtype=dt)
        torch.cuda.synchronize()
        for b in range(P):
            want = arr(c["out"][b], dt)[:counts[b]]
            assert_bits_equal(to_host(d_recvs[b], npdt)[:counts[b]], want, dt, "reduce_scatterv P=%d rank %d" % (P, b))


MPIEXEC = "/opt/conda/bin/mpiexec"
MPI_PROGRAM = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "mpi_baseline")


@pytest.mark.skipif(not (os.path.exists(MPIEXEC) and os.path.exists(MPI_PROGRAM)),
                    reason="needs mpiexec and the built oracle/mpi_baseline")
@pytest.mark.parametrize("P", (2, 3, 4, 5, 8))
def test_live_mpi_allreduce_against_the_gpu(al, P):
    """MPI_Allreduce(MPI_SUM, MPI_FLOAT) run now, on this machine's host cores, over generated inputs
    (uniform[-1,1), seed 1000+rank), against the GPU's combine of the same inputs: equal checksums."""
    import subprocess
    import torch
    for n in (300, 513, (1 << 16) + 1, 1 << 20):
        p = subprocess.run([MPIEXEC, "-n", str(P), MPI_PROGRAM, str(n), "0", "1"], capture_output=True, text=True,
                           timeout=120)
        line = [l for l in p.stdout.splitlines() if l.startswith("{")]
        assert p.returncode == 0 and line, (p.stdout, p.stderr)
        want = json.loads(line[-1])["checksum"]
        ins = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(P)]
        out = torch.empty(n, dtype=torch.float32, device="cuda")
        for r in range(P):
            al.fill(ins[r], "uniform_pm1", 1000 + r)
        order = "tree_binomial" if n * 4 <= 2048 else "tree_dbl"
        al.combine([out], ins, "sum", order=order)
        torch.cuda.synchronize()
        assert "%016x" % oracle.checksum(out.cpu().numpy()) == want, "P=%d n=%d" % (P, n)
