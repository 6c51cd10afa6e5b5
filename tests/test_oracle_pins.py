"""Pins of the CPU oracle against things other than itself: numpy and torch
library arithmetic, brute-force Python restatements of each named order from
its definition, closed forms and invariants."""
import functools
import itertools

import numpy as np
import pytest

import oracle
from util import ALL_DTYPES, FLOAT_DTYPES, INT_DTYPES, assert_bits_equal, ops_of

NP_OF = {"i8": np.int8, "u8": np.uint8, "i16": np.int16, "u16": np.uint16, "i32": np.int32,
         "u32": np.uint32, "i64": np.int64, "u64": np.uint64}


# ---- the two-operand step ----------------------------------------------------

@pytest.mark.parametrize("dtype", INT_DTYPES)
def test_int_step_against_numpy(dtype):
    n = 4096
    a = oracle.fill(n, dtype, "fullrange", 1)
    b = oracle.fill(n, dtype, "fullrange", 2)
    a[:64] = 0
    b[32:96] = 0
    with np.errstate(over="ignore"):
        want = {
            "sum": a + b, "prod": a * b, "min": np.minimum(a, b), "max": np.maximum(a, b),
            "lor": ((a != 0) | (b != 0)).astype(a.dtype), "land": ((a != 0) & (b != 0)).astype(a.dtype),
            "lxor": ((a != 0) ^ (b != 0)).astype(a.dtype), "bor": a | b, "band": a & b, "bxor": a ^ b,
        }
    for op, w in want.items():
        assert oracle.step(a, b, dtype, op).tobytes() == w.astype(a.dtype).tobytes(), op


@pytest.mark.parametrize("dtype", ("f32", "f64"))
def test_fp_step_against_numpy(dtype):
    n = 1 << 16
    a = oracle.fill(n, dtype, "uniform_pm1", 3)
    b = oracle.fill(n, dtype, "uniform_pm1", 4)
    tiny = np.finfo(a.dtype).tiny
    a[:100] *= tiny  # denormal results
    b[:100] *= tiny
    assert oracle.step(a, b, dtype, "sum").tobytes() == (a + b).tobytes()
    assert oracle.step(a, b, dtype, "prod").tobytes() == (a * b).tobytes()
    assert oracle.step(a, b, dtype, "min").tobytes() == np.minimum(a, b).tobytes()
    assert oracle.step(a, b, dtype, "max").tobytes() == np.maximum(a, b).tobytes()


def test_unsupported_pairs():
    # include/aluminum/mpi/utils.hpp:169-269; avg (NCCL path only in the reference) is defined for every type
    for dt in ALL_DTYPES:
        assert oracle.check_op(dt, "avg") == 0
        assert oracle.check_op(dt, 11) != 0
        for op in ("lor", "land", "lxor", "bor", "band", "bxor"):
            assert (oracle.check_op(dt, op) != 0) == (dt in FLOAT_DTYPES)
        for op in ("sum", "prod", "min", "max"):
            assert oracle.check_op(dt, op) == 0
    with pytest.raises(ValueError):
        oracle.step(np.zeros(4, np.float32), np.zeros(4, np.float32), "f32", "band")


# ---- 16-bit floats -----------------------------------------------------------

def trunc_div(a, d):
    """C integer division of a numpy integer array by d, through Python integers."""
    return np.array([abs(int(v)) // d * (1 if v >= 0 else -1) for v in a.tolist()], dtype=a.dtype)


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_avg_is_sum_then_divide(dtype):
    """avg = the sum of the same order, then one division by P: pinned with numpy / torch division of
    the oracle's own sum (itself pinned above) and with closed forms."""
    import torch
    n = 3000
    np_dt = oracle.NP_CARRIER[dtype]
    for P in (1, 2, 3, 7, 8, 64):
        dist = "fullrange" if dtype in INT_DTYPES else "uniform_pm1"
        ins = [oracle.fill(n, dtype, dist, 50 + r) for r in range(P)]
        for order in ("rank_asc", "tree_dbl"):
            s = oracle.combine(ins, dtype, "sum", order)
            got = oracle.combine(ins, dtype, "avg", order)
            if dtype in INT_DTYPES:
                want = trunc_div(s, P)   # truncation toward zero
            elif dtype == "f32":
                want = s / np.float32(P)
            elif dtype == "f64":
                want = s / np.float64(P)
            elif dtype == "f16":
                want = (s.view(np.float16).astype(np.float32) / np.float32(P)).astype(np.float16).view(np.uint16)
            else:  # bf16: widen, fp32 division, torch's round-to-nearest-even narrowing
                wide = torch.from_numpy(s.view(np.int16).copy()).view(torch.bfloat16).float()
                want = (wide / float(P)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
            assert_bits_equal(got, want, dtype, "avg %s P=%d %s" % (dtype, P, order))
            assert_bits_equal(oracle.divide(s, dtype, P), want, dtype, "divide %s P=%d" % (dtype, P))
    # closed forms: equal contributions whose sum is exact average to the contribution itself
    x = oracle.fill(n, dtype, "smallint", 9)
    for P in (2, 4, 5, 8):
        assert_bits_equal(oracle.combine([x] * P, dtype, "avg", "rank_asc"), x, dtype, "avg of equals")
    # truncation toward zero, not flooring: (-7) / 2 = -3; unsigned wraps before it divides
    if dtype in ("i8", "i16", "i32", "i64"):
        a = np.array([-7, 7, -1, 1], dtype=np_dt)
        assert oracle.combine([a, np.zeros(4, np_dt)], dtype, "avg", "rank_asc").tolist() == [-3, 3, 0, 0]
    if dtype == "u8":
        a = np.array([200, 100], dtype=np_dt)
        assert oracle.combine([a, a], dtype, "avg", "rank_asc").tolist() == [(400 % 256) // 2, 100]


def test_f16_widen_all_patterns_against_numpy():
    bits = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.f16_to_f32(bits)
    assert_bits_equal(got, want, "f32", "f16 widen")
    nn = ~np.isnan(want)
    assert got[nn].tobytes() == want[nn].tobytes()


def test_bf16_widen_all_patterns():
    bits = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    want = (bits.astype(np.uint32) << 16).view(np.float32)
    assert oracle.bf16_to_f32(bits).tobytes() == want.tobytes()


def edge_f32():
    """fp32 values around every rounding boundary of both 16-bit formats."""
    out = []
    for hb in (0x0000, 0x0001, 0x03ff, 0x0400, 0x3bff, 0x3c00, 0x7bff, 0x7c00):  # f16 neighbours
        f = int(np.array([hb], np.uint16).view(np.float16).astype(np.float32).view(np.uint32)[0])
        out += [f + d for d in (-0x2000, -0x1001, -0x1000, -0xfff, -1, 0, 1, 0xfff, 0x1000, 0x1001, 0x2000)
                if 0 <= f + d < 2 ** 31]
    for top in (0x0000, 0x0001, 0x007f, 0x0080, 0x3f80, 0x7f7f, 0x7f80):  # bf16 neighbours
        out += [(top << 16) + d for d in (0, 1, 0x7fff, 0x8000, 0x8001, 0xffff)]
    out += [0x33000000, 0x33000001, 0x32ffffff, 0x477fe000, 0x477fefff, 0x477ff000, 0x47800000]
    a = np.array(out, dtype=np.uint32)
    a = np.concatenate([a, a | 0x80000000])
    return a.view(np.float32)


def test_f16_narrow_against_numpy():
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.integers(0, 2 ** 32, 1 << 22, dtype=np.uint64).astype(np.uint32).view(np.float32),
                        edge_f32()])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert oracle.f32_to_f16(x).tobytes() == want.tobytes()


def test_bf16_narrow_against_torch():
    import torch
    rng = np.random.default_rng(6)
    x = np.concatenate([rng.integers(0, 2 ** 32, 1 << 22, dtype=np.uint64).astype(np.uint32).view(np.float32),
                        edge_f32()])
    x = x[~np.isnan(x)]
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert oracle.f32_to_bf16(x).tobytes() == want.tobytes()


def test_nan_stays_nan_when_narrowed():
    nans = np.array([0x7fc00000, 0x7f800001, 0xffc12345, 0x7fffffff, 0xff800100], np.uint32).view(np.float32)
    b = oracle.f32_to_bf16(nans)
    h = oracle.f32_to_f16(nans)
    assert ((b & 0x7fff) > 0x7f80).all() and ((h & 0x7fff) > 0x7c00).all()


@pytest.mark.parametrize("dtype", ("bf16", "f16"))
def test_16bit_step_against_torch(dtype):
    """src/mpi_impl.cpp:61-145: widen, one fp32 operation, narrow."""
    import torch
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float16
    n = 1 << 16
    a = oracle.fill(n, dtype, "normal", 11)
    b = oracle.fill(n, dtype, "uniform_pm1", 12)
    ta = torch.from_numpy(a.view(np.int16)).view(tdt).float()
    tb = torch.from_numpy(b.view(np.int16)).view(tdt).float()
    for op, f in (("sum", ta + tb), ("prod", ta * tb), ("min", torch.minimum(ta, tb)), ("max", torch.maximum(ta, tb))):
        want = f.to(tdt).view(torch.int16).numpy().view(np.uint16)
        assert oracle.step(a, b, dtype, op).tobytes() == want.tobytes(), op


def test_16bit_minmax_operand_choice():
    # std::min(in, inout) / std::max(in, inout): a tie or a NaN inout yields `in`
    pz, nz, nan, one = 0x0000, 0x8000, 0x7fc0, 0x3f80
    inn = np.array([pz, nz, one, nan, one], np.uint16)
    ino = np.array([nz, pz, nan, one, one], np.uint16)
    got_min = oracle.step(ino, inn, "bf16", "min")
    got_max = oracle.step(ino, inn, "bf16", "max")
    assert got_min.tolist()[:3] == [pz, nz, one] and got_max.tolist()[:3] == [pz, nz, one]
    assert (got_min[3] & 0x7fff) > 0x7f80 and (got_max[3] & 0x7fff) > 0x7f80


# ---- named orders from their definitions -------------------------------------

def py_step(op):
    return {"sum": lambda inn, ino: ino + inn, "prod": lambda inn, ino: ino * inn,
            "min": lambda inn, ino: ino if ino < inn else inn,
            "max": lambda inn, ino: ino if ino > inn else inn}[op]


def brute(xs, op, order, start):
    """Value of one element under a named order, from the order's definition."""
    st = py_step(op)
    P = len(xs)
    if order == "rank_asc":
        return functools.reduce(lambda acc, x: st(x, acc), xs[1:], xs[0])
    if order == "pairwise_desc":
        acc = xs[start]
        for k in range(1, P):
            acc = st(xs[(start - k) % P], acc)
        return acc
    if order == "ring":
        acc = xs[start]
        for k in range(1, P):
            acc = st(acc, xs[(start + k) % P])  # the travelling partial is `in`
        return acc
    if order == "tree_binomial":
        v = [xs[(j + start) % P] for j in range(P)]  # ranks counted from the root, with wrap
        d = 1
        while d < P:
            for i in range(0, P - d, 2 * d):
                v[i] = st(v[i + d], v[i])
            d *= 2
        return v[0]
    # tree_dbl / tree_halv
    pof2 = 1 << (P.bit_length() - 1)
    rem = P - pof2
    L = [st(xs[2 * j], xs[2 * j + 1]) for j in range(rem)] + [xs[j + rem] for j in range(rem, pof2)]

    def dbl(v):
        return v[0] if len(v) == 1 else st(dbl(v[len(v) // 2:]), dbl(v[:len(v) // 2]))

    def halv(v, o):
        # the half that holds survivor o keeps its own values and folds in the other half's
        if len(v) == 1:
            return v[0]
        h = len(v) // 2
        if o < h:
            return halv([st(v[i + h], v[i]) for i in range(h)], o)
        return halv([st(v[i], v[i + h]) for i in range(h)], o - h)

    return dbl(L) if order == "tree_dbl" else halv(L, start // 2 if start < 2 * rem else start - rem)


@pytest.mark.parametrize("P", (1, 2, 3, 4, 5, 6, 7, 8, 11, 16))
def test_orders_against_brute_force(P):
    n = 40
    for op, dist in (("sum", "uniform_pm1"), ("prod", "uniform_09_11"), ("max", "uniform_pm1"), ("min", "bool01")):
        # {0, 1} inputs under min: ties everywhere, so the operand roles show
        ins = [oracle.fill(n, "f64", dist, 50 + r) for r in range(P)]
        if dist == "bool01":
            ins = [np.where(a == 0, np.where(np.arange(n) % (r + 2) == 0, -0.0, 0.0), a) for r, a in enumerate(ins)]
        for order in oracle.ORDERS:
            if order in ("tree_rsg", "tree_rsg_spread"):
                continue  # depend on the element's position: see the simulation below
            starts = range(P) if order in ("pairwise_desc", "ring", "tree_binomial", "tree_halv") else (0,)
            for start in starts:
                got = oracle.combine(ins, "f64", op, order, start)
                want = np.array([brute([float(a[i]) for a in ins], op, order, start) for i in range(n)])
                assert got.tobytes() == want.tobytes(), (P, op, order, start)


def simulate_reduce_scatter_gather(ins, dtype, op, spread=False):
    """P ranks exchanging messages: a reduce-scatter by recursive halving of the data at distance 1, 2,
    4, ... (odd ranks among the first 2 * rem hand their data to the even rank below them first; what
    a rank receives is the invec of its step, what it holds the inoutvec), then the blocks gathered from
    their owners.  The vector that a reduce or allreduce of a long message leaves at the root; what the
    count is not a multiple of goes to the last block (MPI_Ireduce, MPI_Iallreduce) or, `spread`, one
    element each to the first blocks (MPI_Reduce, MPI_Allreduce)."""
    P, n = len(ins), ins[0].size
    pof2 = 1 << (P.bit_length() - 1)
    rem = P - pof2
    buf = [a.copy() for a in ins]
    real = [2 * nr if nr < rem else nr + rem for nr in range(pof2)]
    for j in range(rem):
        buf[2 * j] = oracle.step(buf[2 * j], buf[2 * j + 1], dtype, op)
    cnts = [n // pof2] * pof2
    if spread:
        for k in range(n % pof2):
            cnts[k] += 1
    else:
        cnts[-1] = n - (n // pof2) * (pof2 - 1)
    assert sum(cnts) == n
    disps = [sum(cnts[:k]) for k in range(pof2 + 1)]
    lo_hi = {nr: (0, pof2) for nr in range(pof2)}  # the blocks a rank still works on
    mask = 1
    while mask < pof2:
        before = [b.copy() for b in buf]
        for nr in range(pof2):
            lo, hi = lo_hi[nr]
            mid = (lo + hi) // 2
            keep = (lo, mid) if nr < (nr ^ mask) else (mid, hi)
            a, b = disps[keep[0]], disps[keep[1]]
            me, other = real[nr], real[nr ^ mask]
            buf[me][a:b] = oracle.step(before[me][a:b].copy(), before[other][a:b].copy(), dtype, op)
            lo_hi[nr] = keep
        mask *= 2
    out = np.empty_like(ins[0])
    for nr in range(pof2):
        k = lo_hi[nr][0]
        out[disps[k]:disps[k + 1]] = buf[real[nr]][disps[k]:disps[k + 1]]
    return out


def simulate_recursive_halving_reduce_scatter(ins, counts, dtype, op):
    """P ranks exchanging messages: even ranks among the first 2 * rem hand their data to the odd rank
    above them; the survivors exchange halves of the blocks they still work on at distance pof2 / 2, ...,
    1, keeping the half their own blocks lie in (what arrives is the invec); a survivor that stands for
    two ranks hands the even one its block back.  Returns the block each rank ends with."""
    P = len(ins)
    pof2 = 1 << (P.bit_length() - 1)
    rem = P - pof2
    disp = [sum(counts[:b]) for b in range(P + 1)]
    buf = [a.copy() for a in ins]
    real = [2 * nr + 1 if nr < rem else nr + rem for nr in range(pof2)]
    for j in range(rem):
        buf[2 * j + 1] = oracle.step(buf[2 * j + 1], buf[2 * j], dtype, op)
    # the ranks whose blocks survivor nr is responsible for
    owned = [[2 * nr, 2 * nr + 1] if nr < rem else [nr + rem] for nr in range(pof2)]
    lo_hi = {nr: (0, pof2) for nr in range(pof2)}
    d = pof2 // 2
    while d >= 1:
        before = [b.copy() for b in buf]
        for nr in range(pof2):
            lo, hi = lo_hi[nr]
            mid = (lo + hi) // 2
            keep = (lo, mid) if nr < mid else (mid, hi)
            first, last = owned[keep[0]][0], owned[keep[1] - 1][-1]
            a, b = disp[first], disp[last + 1]
            me, other = real[nr], real[nr ^ d]
            buf[me][a:b] = oracle.step(before[me][a:b].copy(), before[other][a:b].copy(), dtype, op)
            lo_hi[nr] = keep
        d //= 2
    out = []
    for b in range(P):
        nr = b // 2 if b < 2 * rem else b - rem
        out.append(buf[real[nr]][disp[b]:disp[b + 1]].copy())
    return out


def specials(n, seed):
    pool = np.array([np.nan, -1.0, 0.0, -0.0, np.inf, -np.inf, 1e-45, 1.0, 3.0e38, 0.3], np.float32)
    idx = np.array([oracle.mix64(seed, i) % pool.size for i in range(n)])
    return pool[idx]


@pytest.mark.parametrize("P", (2, 3, 4, 5, 6, 7, 8, 12, 16, 33))
def test_tree_rsg_against_a_message_passing_simulation(P):
    for n in (P, 64, 67, 300):
        if n < (1 << (P.bit_length() - 1)):
            continue
        for op in ("sum", "min", "max"):
            ins = [specials(n, 900 + r) if op != "sum" else oracle.fill(n, "f32", "uniform_pm1", 900 + r) for r in range(P)]
            for spread in (False, True):
                got = oracle.combine(ins, "f32", op, "tree_rsg_spread" if spread else "tree_rsg")
                want = simulate_reduce_scatter_gather(ins, "f32", op, spread)
                assert_same(got, want, (P, n, op, spread))


@pytest.mark.parametrize("P", (2, 3, 4, 5, 6, 7, 8, 12, 16))
def test_tree_halv_against_a_message_passing_simulation(P):
    counts = [3 + (5 * b) % 4 if b != 1 else 0 for b in range(P)]
    for op in ("sum", "min", "max"):
        ins = [specials(sum(counts), 700 + r) if op != "sum" else oracle.fill(sum(counts), "f32", "uniform_pm1", 700 + r)
               for r in range(P)]
        got = oracle.reduce_scatterv(ins, counts, "f32", op, "tree_halv")
        want = simulate_recursive_halving_reduce_scatter(ins, counts, "f32", op)
        for b in range(P):
            assert_same(got[b], want[b], (P, op, b))


def assert_same(got, want, what):
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all(), (what, np.flatnonzero(~same)[:5])


def test_orders_agree_where_arithmetic_is_exact():
    P, n = 8, 1000
    ins = [oracle.fill(n, "f32", "smallint", 70 + r) for r in range(P)]
    exact = np.sum(np.stack(ins).astype(np.float64), axis=0).astype(np.float32)
    for order in oracle.ORDERS:
        assert oracle.combine(ins, "f32", "sum", order, 0).tobytes() == exact.tobytes()
    ints = [oracle.fill(n, "i32", "fullrange", 80 + r) for r in range(P)]
    with np.errstate(over="ignore"):
        want = functools.reduce(lambda a, b: a + b, ints)
    for order in oracle.ORDERS:
        assert oracle.combine(ints, "i32", "sum", order, 0).tobytes() == want.tobytes()


def test_rank_asc_float32_against_numpy_cumulative_fold():
    P, n = 8, 5000
    ins = [oracle.fill(n, "f32", "uniform_pm1", 1000 + r) for r in range(P)]
    acc = ins[0].copy()
    for r in range(1, P):
        acc = acc + ins[r]  # numpy float32 add: one IEEE rounding per step
    assert oracle.combine(ins, "f32", "sum", "rank_asc").tobytes() == acc.tobytes()
    gen = oracle.combine_generated(P, n, "f32", "sum", "rank_asc", 0, "uniform_pm1", 1000)
    assert gen.tobytes() == acc.tobytes()


def test_bf16_rank_asc_against_torch_fold():
    import torch
    P, n = 8, 4096
    ins = [oracle.fill(n, "bf16", "normal", 2000 + r) for r in range(P)]
    acc = torch.from_numpy(ins[0].view(np.int16)).view(torch.bfloat16)
    for r in range(1, P):
        x = torch.from_numpy(ins[r].view(np.int16)).view(torch.bfloat16)
        acc = (acc.float() + x.float()).to(torch.bfloat16)  # fp32 accumulate, round per step
    want = acc.view(torch.int16).numpy().view(np.uint16)
    assert oracle.combine(ins, "bf16", "sum", "rank_asc").tobytes() == want.tobytes()


def test_schedule_shape():
    for P in range(1, 20):
        for order in oracle.ORDERS:
            pairs, result = oracle.schedule(P, order, 0)
            assert len(pairs) == P - 1
            ins_used = [p[1] for p in pairs]
            assert len(set(ins_used)) == P - 1 and result not in ins_used  # every operand folded once
    with pytest.raises(ValueError):
        oracle.schedule(4, "ring", 4)


# ---- reduce_scatter / allgather layouts --------------------------------------

def test_reduce_scatter_and_allgather_layout():
    P, count = 5, 7
    sends = [np.arange(P * count, dtype=np.int32) + 1000 * r for r in range(P)]
    rs = oracle.reduce_scatter(sends, "i32", "sum", "rank_asc")
    for b in range(P):
        want = sum(s[b * count:(b + 1) * count] for s in sends)
        assert (rs[b] == want).all()
    ag = oracle.allgather([s[:count] for s in sends], "i32")
    for r in range(P):
        assert (ag[r] == np.concatenate([s[:count] for s in sends])).all()


def test_v_variants_layout():
    P = 4
    counts = [3, 0, 5, 2]
    total = sum(counts)
    sends = [np.arange(total, dtype=np.int64) * (r + 1) for r in range(P)]
    rs = oracle.reduce_scatterv(sends, counts, "i64", "sum", "rank_asc")
    displ = np.concatenate([[0], np.cumsum(counts)])
    for b in range(P):
        want = sum(s[displ[b]:displ[b + 1]] for s in sends)
        assert rs[b].size == counts[b] and (rs[b] == want).all()
    displs = [7, 0, 1, 12]  # arbitrary order, with gaps
    pieces = [np.full(counts[q], q + 1, dtype=np.int16) for q in range(P)]
    ag = oracle.allgatherv(pieces, counts, displs, "i16", fill_value=-1)
    want = np.full(14, -1, dtype=np.int16)
    for q in range(P):
        want[displs[q]:displs[q] + counts[q]] = q + 1
    for r in range(P):
        assert (ag[r] == want).all()


# ---- ring ---------------------------------------------------------------------

@pytest.mark.parametrize("P", (1, 2, 3, 4, 8))
@pytest.mark.parametrize("dtype,op", [("bf16", "sum"), ("f32", "prod"), ("f16", "min"), ("i32", "sum")])
def test_ring_literal_equals_closed_form(P, dtype, op):
    for n in (P, 3 * P + 2, 257):
        dist = "normal" if dtype in FLOAT_DTYPES else "fullrange"
        bufs = [oracle.fill(n, dtype, dist, 2000 + r) for r in range(P)]
        outs = {c: oracle.ring_allreduce(bufs, dtype, op, c) for c in (1, 3, 1 << 20)}
        for c, res in outs.items():  # chunk size never changes a bit; all ranks agree
            for r in range(P):
                assert res[r].tobytes() == outs[1][0].tobytes(), (c, r)
        # segment s is the ring-order fold that starts at rank s
        for s in range(P):
            off, ln = oracle.ring_segment(n, P, s)
            want = oracle.combine([b[off:off + ln] for b in bufs], dtype, op, "ring", s)
            assert outs[1][0][off:off + ln].tobytes() == want.tobytes(), s
        segs = [oracle.ring_segment(n, P, s) for s in range(P)]
        assert segs[0][0] == 0 and sum(l for _, l in segs) == n
        assert all(segs[s][0] + segs[s][1] == segs[s + 1][0] for s in range(P - 1))


def test_ring_reduce_scatter_ownership():
    P, n = 4, 64
    bufs = [oracle.fill(n, "f64", "uniform_pm1", 10 + r) for r in range(P)]
    rs = oracle.ring_reduce_scatter(bufs, "f64", "sum", 5)
    for r in range(P):  # rank r ends up owning segment (r+1) mod P
        s = (r + 1) % P
        off, ln = oracle.ring_segment(n, P, s)
        want = oracle.combine([b[off:off + ln] for b in bufs], "f64", "sum", "ring", s)
        assert rs[r][off:off + ln].tobytes() == want.tobytes()


# ---- halo ---------------------------------------------------------------------

@pytest.mark.parametrize("dims,h", [((5, 4, 3), 1), ((6, 7, 8), 2), ((4, 4, 4), 4)])
def test_halo_against_numpy_slicing(dims, h):
    nx, ny, nz = dims
    g = np.random.default_rng(1).random((nz + 2 * h, ny + 2 * h, nx + 2 * h))
    I = {0: slice(h, None), 1: slice(None, -h)}
    interior = lambda n: slice(h, h + n)
    src = {0: (interior(nz), interior(ny), slice(h, 2 * h)), 1: (interior(nz), interior(ny), slice(nx, nx + h)),
           2: (interior(nz), slice(h, 2 * h), interior(nx)), 3: (interior(nz), slice(ny, ny + h), interior(nx)),
           4: (slice(h, 2 * h), interior(ny), interior(nx)), 5: (slice(nz, nz + h), interior(ny), interior(nx))}
    dst = {0: (interior(nz), interior(ny), slice(0, h)), 1: (interior(nz), interior(ny), slice(h + nx, nx + 2 * h)),
           2: (interior(nz), slice(0, h), interior(nx)), 3: (interior(nz), slice(h + ny, ny + 2 * h), interior(nx)),
           4: (slice(0, h), interior(ny), interior(nx)), 5: (slice(h + nz, nz + 2 * h), interior(ny), interior(nx))}
    for f in range(6):
        buf = oracle.halo_pack(g.reshape(-1), nx, ny, nz, h, f)
        assert buf.size == oracle.halo_face_elems(nx, ny, nz, h, f)
        assert buf.tobytes() == np.ascontiguousarray(g[src[f]]).tobytes(), f
        out = oracle.halo_unpack(g.reshape(-1), buf, nx, ny, nz, h, f).reshape(g.shape)
        want = g.copy()
        want[dst[f]] = g[src[f]]
        assert out.tobytes() == want.tobytes(), f
    del I


# ---- generator ------------------------------------------------------------------

def test_generator_properties():
    n = 1 << 16
    u = oracle.fill(n, "f64", "uniform_pm1", 1000)
    assert -1.0 <= u.min() < -0.99 and 0.99 < u.max() <= 1.0 and abs(u.mean()) < 0.02
    assert len(np.unique(u)) == n
    p = oracle.fill(n, "f32", "uniform_09_11", 1000)
    assert 0.9 <= p.min() and p.max() <= np.float32(1.1) and abs(p.mean() - 1.0) < 0.01
    z = oracle.bf16_to_f32(oracle.fill(n, "bf16", "normal", 2000))
    assert abs(z.mean()) < 0.02 and abs(z.std() - 1.0) < 0.02
    b = oracle.fill(n, "u8", "bool01", 3000)
    assert set(np.unique(b)) == {0, 1} and abs(b.mean() - 0.5) < 0.02
    i = oracle.fill(n, "i64", "fullrange", 3000)
    assert i.min() < -2 ** 62 and i.max() > 2 ** 62
    # counter-based: any slice can be regenerated from its offset
    assert oracle.fill(100, "f32", "uniform_pm1", 7, 500).tobytes() == oracle.fill(600, "f32", "uniform_pm1", 7)[500:].tobytes()
    assert oracle.fill(64, "f32", "uniform_pm1", 7).tobytes() != oracle.fill(64, "f32", "uniform_pm1", 8).tobytes()
    # the fp32 draw is the fp64 draw narrowed once
    assert oracle.fill(n, "f32", "uniform_pm1", 1000).tobytes() == u.astype(np.float32).tobytes()
