"""Helpers shared by the test files: numpy <-> device carriers, comparisons."""
import numpy as np

SIGNED_VIEW = {np.dtype(np.uint16): np.int16, np.dtype(np.uint32): np.int32,
               np.dtype(np.uint64): np.int64}

FLOAT_DTYPES = ("f16", "bf16", "f32", "f64")
INT_DTYPES = ("i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64")
ALL_DTYPES = INT_DTYPES + FLOAT_DTYPES
FP_OPS = ("sum", "prod", "min", "max", "avg")
INT_OPS = ("sum", "prod", "min", "max", "lor", "land", "lxor", "bor", "band", "bxor", "avg")
ORDERS = ("rank_asc", "tree_dbl", "tree_halv", "pairwise_desc", "ring", "tree_binomial", "tree_rsg",
          "tree_rsg_spread")


def floor_pow2(p):
    q = 1
    while 2 * q <= p:
        q *= 2
    return q


def mpich_order(coll, dtype, count, P, root=0, total=None, blocking=False):
    """(order, start) that MPICH 3.3.2 on one host follows for the call the reference makes - what the
    golden vectors in tests/golden establish.  Rooted reduce and allreduce (the latter is a reduce to
    rank 0 followed by a broadcast): binomial tree to the root over the ranks counted from it, up to
    2048 bytes, for fewer elements than the largest power of two of ranks, and for every user-defined
    operation (fp16 / bf16); above that a reduce-scatter by recursive halving plus gather, whatever the
    root - MPI_Ireduce and MPI_Iallreduce (which the host-transfer backend and the MPI backend's
    non-blocking calls make) leave what the count is not a multiple of to the last block, MPI_Reduce and
    MPI_Allreduce (`blocking`: the MPI backend's blocking calls) spread it over the first blocks.
    Reduce_scatter (block or not): recursive halving below 512 KiB in all, pairwise exchange from
    there on; `start` is then added per receiving rank by the collective itself."""
    es = {"f16": 2, "bf16": 2, "f32": 4, "f64": 8}.get(dtype) or int("".join(c for c in dtype if c.isdigit())) // 8
    if coll in ("allreduce", "reduce"):
        r = root if coll == "reduce" else 0
        if dtype in ("f16", "bf16") or count * es <= 2048 or count < floor_pow2(P):
            return "tree_binomial", r
        return ("tree_rsg_spread" if blocking else "tree_rsg"), 0
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


_POOL = np.array([0x7fc00000, 0xbf800000, 0x00000000, 0x80000000, 0x7f800000, 0xff800000, 0x00000001, 0x80000001,
                  0x3f800000, 0x7f7fffff, 0x00800000, 0x00400000, 0x3e99999a], dtype=np.uint32)


def _fin64(z):
    z = z ^ (z >> np.uint64(30))
    z = z * np.uint64(0xBF58476D1CE4E5B9)
    z = z ^ (z >> np.uint64(27))
    z = z * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def mix64(seed, idx):
    """The generator's hash (oracle.mix64) over an array of indices."""
    g = np.uint64(0x9E3779B97F4A7C15)
    with np.errstate(over="ignore"):
        return _fin64(_fin64(np.uint64(seed) + g) + (idx.astype(np.uint64) + np.uint64(1)) * g)


def planted_specials(n, dtype, rank):
    """The inputs that the golden generator plants for more than two ranks (tests/golden/mpich_golden.c,
    plant_specials_many): element i of `rank` is drawn from a pool of NaN, zeros of both signs, infinities,
    denormals and a few ordinary values by a fixed rule; every fourth element is a zero of one sign or the other."""
    import oracle
    i = np.arange(n, dtype=np.uint64)
    h = mix64(77, i * np.uint64(64) + np.uint64(rank))
    u = _POOL[(h % np.uint64(len(_POOL))).astype(np.int64)]
    fourth = (i % np.uint64(4)) == 0
    neg = fourth & (((h >> np.uint64(32)) % np.uint64(3)) == 0)
    u = np.where(fourth, np.where(neg, np.uint32(0x80000000), np.uint32(0)), u).astype(np.uint32)
    f = u.view(np.float32)
    if dtype == "f32":
        return f.copy()
    if dtype == "f64":
        return f.astype(np.float64)
    return oracle.f32_to_bf16(f) if dtype == "bf16" else oracle.f32_to_f16(f)
