"""The CPU oracle against the MPICH golden vectors in tests/golden.

The vectors were produced by MPI_Allreduce / MPI_Reduce_scatter_block of MPICH
3.3.2, the calls the reference's MPI backend forwards to
(include/aluminum/mpi/allreduce.hpp:38-44, mpi/reduce_scatter.hpp:40-46).
They pin the two-operand step of every native type (including NaN, signed
zeros, infinities and denormals), and which named order the reference's
result follows for which collective and message size."""
import glob
import gzip
import json
import os

import numpy as np
import pytest

import oracle
from util import assert_bits_equal

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "mpich_P*.json.gz")))


def load(path):
    with gzip.open(path, "rt") as f:
        return json.load(f)


def arr(hexstr, dtype):
    return np.frombuffer(bytes.fromhex(hexstr), dtype=oracle.NP_CARRIER[dtype]).copy()


def test_fixtures_present():
    assert len(GOLDEN) == 6
    for p in GOLDEN:
        assert "MPICH Version" in load(p)["mpi"]


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-8] for p in GOLDEN])
def test_allreduce_vectors(path):
    doc = load(path)
    P = doc["P"]
    seen = 0
    for c in doc["cases"]:
        if c["coll"] != "allreduce":
            continue
        dt, op, n = c["dtype"], c["op"], c["n"]
        ins = [arr(h, dt) for h in c["in"]]
        outs = [arr(h, dt) for h in c["out"]]
        assert len(ins) == P and ins[0].size == n
        if c["note"] != "specials":
            # the committed inputs are what the generator makes
            for r in range(P):
                assert oracle.fill(n, dt, c["dist"], c["seed_base"] + r).tobytes() == ins[r].tobytes()
        # MPICH 3.3.2 on one host: binomial tree up to 2048 bytes, else the
        # pre-fold + distance-doubling tree
        order = "tree_binomial" if n * ins[0].itemsize <= 2048 else "tree_dbl"
        want = outs[0]
        got = oracle.combine(ins, dt, op, order)
        assert_bits_equal(got, want, dt, "P=%d %s %s n=%d %s" % (P, dt, op, n, c["note"]))
        for r in range(1, P):  # every rank received the same bits
            assert_bits_equal(outs[r], want, dt, "rank %d" % r)
        seen += 1
    assert seen >= 12


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-8] for p in GOLDEN])
def test_reduce_scatter_vectors(path):
    doc = load(path)
    P = doc["P"]
    seen = 0
    for c in doc["cases"]:
        if c["coll"] != "reduce_scatter":
            continue
        dt, op, count = c["dtype"], c["op"], c["n"]
        if "in" in c:
            ins = [arr(h, dt) for h in c["in"]]
            outs = [arr(h, dt) for h in c["out"]]
            got = oracle.reduce_scatter(ins, dt, op, "tree_halv")  # short: recursive halving
            for r in range(P):
                assert_bits_equal(got[r], outs[r], dt, "reduce_scatter short P=%d rank %d" % (P, r))
        else:
            # long: pairwise exchange, rank r folds x_r, x_{r-1}, ... ; outputs kept as checksums
            for r in range(P):
                got = oracle.combine_generated(P, count, dt, op, "pairwise_desc", r, c["dist"],
                                               c["seed_base"], r * count)
                assert "%016x" % oracle.checksum(got) == c["out_checksum"][r], (P, r)
                assert_bits_equal(got[:8], arr(c["out_head"][r], dt), dt, "head")
        seen += 1
    assert seen >= 4


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-8] for p in GOLDEN])
def test_reduce_scatterv_vectors(path):
    """MPI_Reduce_scatter with uneven counts (one of them zero): distance-halving tree."""
    doc = load(path)
    P = doc["P"]
    cases = [c for c in doc["cases"] if c["coll"] == "reduce_scatterv"]
    assert len(cases) == 2
    for c in cases:
        dt, counts = c["dtype"], c["counts"]
        ins = [arr(h, dt) for h in c["in"]]
        outs = [arr(h, dt) for h in c["out"]]
        assert ins[0].size == sum(counts)
        got = oracle.reduce_scatterv(ins, counts, dt, c["op"], "tree_halv")
        for b in range(P):
            assert_bits_equal(got[b], outs[b][:counts[b]], dt, "reduce_scatterv P=%d rank %d" % (P, b))


def test_orders_are_distinguishable():
    """The vectors really separate the orders: a wrong order fails them."""
    doc = load([p for p in GOLDEN if p.endswith("P8.json.gz")][0])
    c = [c for c in doc["cases"] if c["coll"] == "allreduce" and c["dtype"] == "f32" and c["op"] == "sum"
         and c["note"] == "long message"][0]
    ins = [arr(h, "f32") for h in c["in"]]
    want = arr(c["out"][0], "f32")
    match = {o: int((oracle.combine(ins, "f32", "sum", o).view(np.uint32) == want.view(np.uint32)).sum())
             for o in ("rank_asc", "tree_dbl", "tree_halv", "ring")}
    assert match["tree_dbl"] == want.size
    assert match["rank_asc"] < 0.8 * want.size and match["tree_halv"] < 0.8 * want.size


def test_two_operand_step_specials():
    """NaN / signed-zero / infinity behaviour of MPI_MIN, MPI_MAX, MPI_SUM, MPI_PROD."""
    doc = load([p for p in GOLDEN if p.endswith("P2.json.gz")][0])
    cases = [c for c in doc["cases"] if c["note"] == "specials"]
    assert len(cases) == 8
    for c in cases:
        dt, op = c["dtype"], c["op"]
        x0, x1 = (arr(h, dt) for h in c["in"])
        want = arr(c["out"][0], dt)
        # rank 0 keeps x0 as inoutvec and receives x1 as invec
        got = oracle.step(x0, x1, dt, op)
        assert_bits_equal(got, want, dt, "%s %s" % (dt, op))
        if op in ("min", "max"):  # a tie or a NaN yields the invec element, bit for bit
            k = 3  # +0 against -0
            assert got[k].tobytes() == x1[k].tobytes() == want[k].tobytes()
