"""The CPU oracle against the MPICH golden vectors in tests/golden.

The vectors were produced by MPI_Allreduce / MPI_Reduce / MPI_Reduce_scatter_block /
MPI_Reduce_scatter of MPICH 3.3.2, the calls the reference's MPI backend forwards to
(include/aluminum/mpi/allreduce.hpp:38-44, mpi/reduce.hpp:41-49, mpi/reduce_scatter.hpp:40-46)
and whose non-blocking in-place forms its host-transfer backend makes
(include/aluminum/ht/allreduce.hpp:76-79, ht/reduce.hpp:72-82, ht/reduce_scatter.hpp:71-74,
ht/reduce_scatterv.hpp:76-79).  They pin the two-operand step of every native type (including
NaN, signed zeros, infinities and denormals), which named order the reference's result follows
for which collective, root, message size and kind of operation, and - through the cases with
special values planted in every operand position - which operand of every pair of the order is
the one a tie or a NaN lets through."""
import glob
import gzip
import json
import os

import numpy as np
import pytest

import oracle
from util import assert_bits_equal, mpich_order, planted_specials

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "mpich_P*.json.gz")),
                key=lambda p: int(os.path.basename(p)[7:-8]))
IDS = [os.path.basename(p)[:-8] for p in GOLDEN]


def load(path):
    with gzip.open(path, "rt") as f:
        return json.load(f)


def arr(hexstr, dtype):
    return np.frombuffer(bytes.fromhex(hexstr), dtype=oracle.NP_CARRIER[dtype]).copy()


def inputs_of(c, P, n):
    """The P input buffers of a case: the committed ones, or the generator's where the fixture
    does not repeat them."""
    if "in" in c:
        return [arr(h, c["dtype"]) for h in c["in"]]
    if c["note"] == "specials":
        return [planted_specials(n, c["dtype"], r) for r in range(P)]
    return [oracle.fill(n, c["dtype"], c["dist"], c["seed_base"] + r) for r in range(P)]


def lean(P):
    """From 32 ranks on a fixture holds a small set of cases, outputs only, and one output for an allreduce
    (with the generator's word that every rank received the same bytes)."""
    return P >= 32


def test_fixtures_present():
    assert [load(p)["P"] for p in GOLDEN] == [2, 3, 4, 5, 7, 8, 16, 33, 48, 64]
    for p in GOLDEN:
        doc = load(p)
        assert "MPICH Version" in doc["mpi"]
        # the non-blocking in-place form, which the host-transfer backend calls, returned the
        # same bytes as the blocking one, or the fixture holds what it returned: long Allreduce and
        # Reduce messages of native floats, where the two forms cut their blocks differently
        for c in doc["cases"]:
            if not c["nonblocking_in_place_same"]:
                assert c["coll"] in ("allreduce", "reduce") and c["note"] == "specials", c["coll"]
                assert c["dtype"] in ("f32", "f64") and c["n"] * int(c["dtype"][1:]) // 8 > 2048
                assert "out_nonblocking" in c and c.get("nonblocking_all_ranks_same", True)


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_allreduce_vectors(path):
    doc = load(path)
    P = doc["P"]
    seen = halves = 0
    for c in doc["cases"]:
        if c["coll"] != "allreduce":
            continue
        dt, op, n = c["dtype"], c["op"], c["n"]
        ins = inputs_of(c, P, n)
        outs = [arr(h, dt) for h in c["out"]]
        assert len(ins) == P and ins[0].size == n
        if "in" in c and c["note"] != "specials":
            # the committed inputs are what the generator makes
            for r in range(P):
                assert oracle.fill(n, dt, c["dist"], c["seed_base"] + r).tobytes() == ins[r].tobytes()
        if "in" in c and c["note"] == "specials" and P > 2:
            # ... and the planted ones follow the rule that the long cases, which do not repeat them, rely on
            for r in range(P):
                assert planted_specials(n, dt, r).tobytes() == ins[r].tobytes(), (P, dt, n, r)
        # MPI_Allreduce, and MPI_Iallreduce (the same bytes where the fixture holds one output only)
        want = outs[0]
        for blocking in (True, False):
            order, start = mpich_order("allreduce", dt, n, P, blocking=blocking)
            got = oracle.combine(ins, dt, op, order, start)
            ref = want if blocking else arr(c.get("out_nonblocking", c["out"][0]), dt)
            assert_bits_equal(got, ref, dt, "P=%d %s %s n=%d %s (%s)" % (P, dt, op, n, c["note"], order))
        if lean(P):
            assert len(outs) == 1 and c["all_ranks_same"] is True
        else:
            assert len(outs) == P
        for r in range(1, len(outs)):  # every rank received the same bits
            assert outs[r].tobytes() == want.tobytes(), "rank %d" % r
        seen += 1
        halves += dt in ("f16", "bf16")
    assert (seen >= 7 and halves >= 1) if lean(P) else (seen >= 12 and halves >= 6)


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_reduce_vectors(path):
    """MPI_Reduce to the first, second and last rank, below and above 2048 bytes, and at 1 MiB."""
    doc = load(path)
    P = doc["P"]
    seen, roots, orders = 0, set(), set()
    for c in doc["cases"]:
        if c["coll"] != "reduce":
            continue
        dt, op, n, root = c["dtype"], c["op"], c["n"], c["root"]
        for blocking in (True, False):  # MPI_Reduce, MPI_Ireduce
            order, start = mpich_order("reduce", dt, n, P, root, blocking=blocking)
            what = "P=%d %s %s n=%d root %d %s (%s)" % (P, dt, op, n, root, c["note"], order)
            if "out" in c:
                got = oracle.combine(inputs_of(c, P, n), dt, op, order, start)
                ref = c["out"] if blocking else c.get("out_nonblocking", c["out"])
                assert_bits_equal(got, arr(ref, dt), dt, what)
            else:
                assert c["nonblocking_in_place_same"]
                got = oracle.combine_generated(P, n, dt, op, order, start, c["dist"], c["seed_base"])
                assert "%016x" % oracle.checksum(got) == c["out_checksum"], what
                assert_bits_equal(got[:8], arr(c["out_head"], dt), dt, what)
            orders.add(order)
        seen += 1
        roots.add(root)
    assert seen >= (12 if lean(P) else 30) and roots == {0, 1, P - 1}
    assert orders == {"tree_binomial", "tree_rsg", "tree_rsg_spread"}


@pytest.mark.parametrize("path", GOLDEN, ids=IDS)
def test_reduce_scatter_vectors(path):
    doc = load(path)
    P = doc["P"]
    seen = 0
    for c in doc["cases"]:
        if c["coll"] != "reduce_scatter":
            continue
        dt, op, count = c["dtype"], c["op"], c["n"]
        order, _ = mpich_order("reduce_scatter", dt, count, P)
        if "out" in c:
            assert order == "tree_halv"  # short: recursive halving
            ins = inputs_of(c, P, P * count)
            outs = [arr(h, dt) for h in c["out"]]
            got = oracle.reduce_scatter(ins, dt, op, order)
            for r in range(P):
                assert_bits_equal(got[r], outs[r], dt, "reduce_scatter short P=%d %s rank %d" % (P, dt, r))
        else:
            # long: pairwise exchange from 512 KiB in all, rank r folds x_r, x_{r-1}, ... ; outputs kept as checksums
            assert order == ("pairwise_desc" if P * count * oracle.dtype_size(dt) >= (512 << 10) else "tree_halv")
            planted = inputs_of(c, P, P * count) if c["note"] == "specials" else None
            for r in range(P):
                if planted:
                    got = oracle.combine([a[r * count:(r + 1) * count] for a in planted], dt, op, order, r)
                else:
                    got = oracle.combine_generated(P, count, dt, op, order, r, c["dist"], c["seed_base"], r * count)
                # (a min / max result is one of its operands bit for bit, the one planted NaN included)
                assert "%016x" % oracle.checksum(got) == c["out_checksum"][r], (P, dt, r, c["note"])
                assert_bits_equal(got[:8], arr(c["out_head"][r], dt), dt, "head")
        seen += 1
    assert seen >= (3 if lean(P) else 8)


@pytest.mark.parametrize("path", [p for p in GOLDEN if not lean(load(p)["P"])],
                         ids=[i for p, i in zip(GOLDEN, IDS) if not lean(load(p)["P"])])
def test_reduce_scatterv_vectors(path):
    """MPI_Reduce_scatter with uneven counts (one of them zero), below and above 512 KiB in all."""
    doc = load(path)
    P = doc["P"]
    cases = [c for c in doc["cases"] if c["coll"] == "reduce_scatterv"]
    assert len(cases) == 8
    for c in cases:
        dt, counts, total = c["dtype"], c["counts"], c["n"]
        assert total == sum(counts)
        order, _ = mpich_order("reduce_scatterv", dt, 0, P, total=total)
        if "out" in c:
            assert order == "tree_halv"
            ins = inputs_of(c, P, total)
            outs = [arr(h, dt) for h in c["out"]]
            got = oracle.reduce_scatterv(ins, counts, dt, c["op"], order)
            for b in range(P):
                assert_bits_equal(got[b], outs[b][:counts[b]], dt, "reduce_scatterv P=%d rank %d" % (P, b))
        else:
            assert order == "pairwise_desc"
            displ = 0
            for b in range(P):
                got = oracle.combine_generated(P, counts[b], dt, c["op"], order, b, c["dist"], c["seed_base"], displ)
                assert "%016x" % oracle.checksum(got) == c["out_checksum"][b], (P, dt, b)
                if counts[b]:
                    assert_bits_equal(got[:8], arr(c["out_head"][b], dt), dt, "head")
                displ += counts[b]


def test_orders_are_distinguishable():
    """The vectors really separate the orders: a wrong order, or a wrong root, fails them."""
    doc = load([p for p in GOLDEN if p.endswith("P5.json.gz")][0])
    c = [c for c in doc["cases"] if c["coll"] == "allreduce" and c["dtype"] == "f32" and c["op"] == "sum"
         and c["note"] == "long message"][0]
    ins = inputs_of(c, 5, c["n"])
    want = arr(c["out"][0], "f32")
    match = {o: int((oracle.combine(ins, "f32", "sum", o).view(np.uint32) == want.view(np.uint32)).sum())
             for o in ("rank_asc", "tree_dbl", "tree_rsg", "tree_halv", "ring", "tree_binomial")}
    assert match["tree_rsg"] == want.size == match["tree_dbl"]  # the same tree; operand roles differ
    assert all(match[o] < 0.8 * want.size for o in ("rank_asc", "tree_halv", "ring", "tree_binomial"))
    c = [c for c in doc["cases"] if c["coll"] == "reduce" and c["dtype"] == "f32" and c["op"] == "sum"
         and c["note"] == "short message" and c["root"] == 4][0]
    ins = inputs_of(c, 5, c["n"])
    want = arr(c["out"], "f32")
    assert oracle.combine(ins, "f32", "sum", "tree_binomial", 4).tobytes() == want.tobytes()
    assert oracle.combine(ins, "f32", "sum", "tree_binomial", 0).tobytes() != want.tobytes()


def test_specials_separate_the_operand_roles():
    """With NaNs and zeros of both signs in every position, min / max tell which operand of a pair is
    the inoutvec: the doubling tree with fixed roles gets the sums right and the minima wrong, and so
    does the right tree over the wrong blocks."""
    doc = load([p for p in GOLDEN if p.endswith("P8.json.gz")][0])
    cases = [c for c in doc["cases"] if c["coll"] == "allreduce" and c["note"] == "specials" and c["dtype"] == "f32"
             and c["n"] > 512]
    assert {c["op"] for c in cases} == {"sum", "prod", "min", "max"}
    for c in cases:
        ins = inputs_of(c, 8, c["n"])
        want = arr(c["out"][0], "f32")
        assert_bits_equal(oracle.combine(ins, "f32", c["op"], "tree_rsg_spread"), want, "f32", c["op"])
        fixed = oracle.combine(ins, "f32", c["op"], "tree_dbl")
        same = (fixed.view(np.uint32) == want.view(np.uint32)) | (np.isnan(fixed) & np.isnan(want))
        assert same.all() == (c["op"] in ("sum", "prod")), c["op"]
        # ... and where the blocks are cut: 523 elements are not a multiple of 8, and the non-blocking
        # call, which leaves the three over to the last block, returned other minima
        other = oracle.combine(ins, "f32", c["op"], "tree_rsg")
        same = (other.view(np.uint32) == want.view(np.uint32)) | (np.isnan(other) & np.isnan(want))
        assert same.all() == (c["op"] in ("sum", "prod")), c["op"]
        if c["op"] in ("min", "max"):
            assert_bits_equal(other, arr(c["out_nonblocking"], "f32"), "f32", c["op"])


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
