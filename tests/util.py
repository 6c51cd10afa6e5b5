"""Helpers shared by the test files: numpy <-> device carriers, comparisons."""
import numpy as np

SIGNED_VIEW = {np.dtype(np.uint16): np.int16, np.dtype(np.uint32): np.int32,
               np.dtype(np.uint64): np.int64}

FLOAT_DTYPES = ("f16", "bf16", "f32", "f64")
INT_DTYPES = ("i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64")
ALL_DTYPES = INT_DTYPES + FLOAT_DTYPES
FP_OPS = ("sum", "prod", "min", "max", "avg")
INT_OPS = ("sum", "prod", "min", "max", "lor", "land", "lxor", "bor", "band", "bxor", "avg")
ORDERS = ("rank_asc", "tree_dbl", "tree_halv", "pairwise_desc", "ring", "tree_binomial", "tree_rsg")


def floor_pow2(p):
    q = 1
    while 2 * q <= p:
        q *= 2
    return q


def mpich_order(coll, dtype, count, P, root=0, total=None):
    """(order, start) that MPICH 3.3.2 on one host follows for the call the reference makes - what the
    golden vectors in tests/golden establish.  Rooted reduce and allreduce (the latter is a reduce to
    rank 0 followed by a broadcast): binomial tree to the root over the ranks counted from it, up to
    2048 bytes, for fewer elements than the largest power of two of ranks, and for every user-defined
    operation (fp16 / bf16); above that a reduce-scatter by recursive halving plus gather, whatever the
    root.  Reduce_scatter (block or not): recursive halving below 512 KiB in all, pairwise exchange from
    there on; `start` is then added per receiving rank by the collective itself."""
    es = {"f16": 2, "bf16": 2, "f32": 4, "f64": 8}.get(dtype) or int("".join(c for c in dtype if c.isdigit())) // 8
    if coll in ("allreduce", "reduce"):
        r = root if coll == "reduce" else 0
        if dtype in ("f16", "bf16") or count * es <= 2048 or count < floor_pow2(P):
            return "tree_binomial", r
        return "tree_rsg", 0
    if coll in ("reduce_scatter", "reduce_scatterv"):
        total = count * P if total is None else total
        return ("tree_halv" if total * es < (512 << 10) else "pairwise_desc"), 0
    raise ValueError(coll)


def ops_of(dtype):
    return FP_OPS if dtype in FLOAT_DTYPES else INT_OPS


def to_dev(a):
    """numpy array -> torch tensor on the GPU holding the same bytes."""
    import torch
    a = np.ascontiguousarray(a)
    if a.dtype in SIGNED_VIEW:
        a = a.view(SIGNED_VIEW[a.dtype])
    return torch.from_numpy(a.copy()).cuda()


def to_host(t, np_dtype):
    """torch tensor -> numpy array of `np_dtype` holding the same bytes."""
    return t.cpu().numpy().view(np_dtype)


def dev_empty(n, np_dtype):
    import torch
    return to_dev(np.zeros(n, dtype=np_dtype)) if n else torch.empty(0, device="cuda")


def nan_mask(a, dtype):
    """True where element is a NaN of its float type (bit patterns for 16-bit)."""
    if dtype == "f32" or dtype == "f64":
        return np.isnan(a)
    if dtype == "bf16":
        return (a.view(np.uint16) & 0x7fff) > 0x7f80
    if dtype == "f16":
        return (a.view(np.uint16) & 0x7fff) > 0x7c00
    return np.zeros(a.shape, bool)


def assert_bits_equal(got, want, dtype, what=""):
    """Bit-exact equality, except that two NaNs of any payload count as equal."""
    got = np.ascontiguousarray(got)
    want = np.ascontiguousarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    gb = got.view(np.uint8).reshape(got.size, -1) if got.size else got.view(np.uint8)
    wb = want.view(np.uint8).reshape(want.size, -1) if want.size else want.view(np.uint8)
    same = (gb == wb).all(axis=-1) if got.size else np.ones(0, bool)
    if dtype in FLOAT_DTYPES:
        same = same | (nan_mask(got.reshape(-1), dtype) & nan_mask(want.reshape(-1), dtype))
    if not same.all():
        bad = np.flatnonzero(~same)
        i = int(bad[0])
        raise AssertionError("%s: %d of %d elements differ; first at %d: got %r want %r" % (
            what, bad.size, got.size, i, got.reshape(-1)[i], want.reshape(-1)[i]))
