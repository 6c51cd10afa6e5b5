"""ctypes front-end of the CPU oracle (``liboracle.so``).

TEST INFRASTRUCTURE ONLY.  The oracle is the checker for the GPU library: only
the test-suite, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` import this module.  Nothing in ``aluminum_amd`` may.

Arrays cross as numpy arrays; 16-bit floats travel as ``uint16`` bit patterns.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

DTYPES = ["i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64", "f16", "bf16", "f32", "f64"]
OPS = ["sum", "prod", "min", "max", "lor", "land", "lxor", "bor", "band", "bxor", "avg"]
ORDERS = {"rank_asc": 0, "tree_dbl": 1, "tree_halv": 2, "pairwise_desc": 3, "ring": 4,
          "tree_binomial": 5, "tree_rsg": 6, "tree_rsg_spread": 7}
DISTS = {"uniform_pm1": 0, "uniform_09_11": 1, "uniform_01": 2, "fullrange": 3, "bool01": 4,
         "normal": 5, "smallint": 6}

# numpy carrier type of every dtype (f16 / bf16 are carried as raw uint16)
NP_CARRIER = {
    "i8": np.int8, "u8": np.uint8, "i16": np.int16, "u16": np.uint16, "i32": np.int32,
    "u32": np.uint32, "i64": np.int64, "u64": np.uint64, "f16": np.uint16, "bf16": np.uint16,
    "f32": np.float32, "f64": np.float64,
}


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        vp, sz, i, u64 = C.c_void_p, C.c_size_t, C.c_int, C.c_uint64
        L.alo_dtype_size.restype = sz
        L.alo_dtype_size.argtypes = [i]
        L.alo_check_op.argtypes = [i, i]
        L.alo_mix64.restype = u64
        L.alo_mix64.argtypes = [u64, u64]
        L.alo_fill.restype = None
        L.alo_fill.argtypes = [vp, sz, i, i, u64, u64]
        for name in ("alo_f32_to_bf16_array", "alo_f32_to_f16_array", "alo_bf16_to_f32_array",
                     "alo_f16_to_f32_array"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, vp, sz]
        L.alo_step.argtypes = [vp, vp, sz, i, i]
        L.alo_divide.argtypes = [vp, sz, i, i]
        L.alo_schedule.argtypes = [i, i, i, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        L.alo_combine.argtypes = [vp, C.POINTER(vp), i, sz, i, i, i, i]
        L.alo_combine_generated.argtypes = [vp, i, sz, i, i, i, i, i, u64, u64]
        L.alo_reduce_scatter.argtypes = [C.POINTER(vp), C.POINTER(vp), i, sz, i, i, i]
        L.alo_allgather.argtypes = [C.POINTER(vp), C.POINTER(vp), i, sz, i]
        L.alo_reduce_scatterv.argtypes = [C.POINTER(vp), C.POINTER(vp), i, C.POINTER(sz), i, i, i]
        L.alo_allgatherv.argtypes = [C.POINTER(vp), C.POINTER(vp), i, C.POINTER(sz), C.POINTER(sz), i]
        L.alo_ring_segment.restype = None
        L.alo_ring_segment.argtypes = [sz, i, i, C.POINTER(sz), C.POINTER(sz)]
        L.alo_ring_allreduce.argtypes = [C.POINTER(vp), i, sz, i, i, sz]
        L.alo_ring_reduce_scatter.argtypes = [C.POINTER(vp), i, sz, i, i, sz]
        L.alo_ring_allgather.argtypes = [C.POINTER(vp), i, sz, i, sz]
        L.alo_halo_face_elems.restype = sz
        L.alo_halo_face_elems.argtypes = [sz, sz, sz, sz, i]
        L.alo_halo_pack.argtypes = [vp, vp, sz, sz, sz, sz, i, sz]
        L.alo_halo_unpack.argtypes = [vp, vp, sz, sz, sz, sz, i, sz]
        L.alo_checksum.restype = u64
        L.alo_checksum.argtypes = [vp, sz]
        L.alo_num_threads.restype = i
        L.alo_set_num_threads.restype = None
        L.alo_set_num_threads.argtypes = [i]
        _lib = L
    return _lib


def _dt(dtype):
    return DTYPES.index(dtype) if isinstance(dtype, str) else int(dtype)


def _op(op):
    return OPS.index(op) if isinstance(op, str) else int(op)


def _order(order):
    return ORDERS[order] if isinstance(order, str) else int(order)


def _dist(dist):
    return DISTS[dist] if isinstance(dist, str) else int(dist)


def _ptr(a):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def _ptr_array(arrays):
    arr = (C.c_void_p * len(arrays))()
    for k, a in enumerate(arrays):
        assert a.flags["C_CONTIGUOUS"]
        arr[k] = a.ctypes.data
    return arr


def dtype_size(dtype):
    return lib().alo_dtype_size(_dt(dtype))


def check_op(dtype, op):
    return lib().alo_check_op(_dt(dtype), _op(op))


def mix64(seed, idx):
    return lib().alo_mix64(seed, idx)


def fill(n, dtype, dist, seed, idx0=0):
    out = np.empty(n, dtype=NP_CARRIER[DTYPES[_dt(dtype)]])
    lib().alo_fill(_ptr(out), n, _dt(dtype), _dist(dist), seed, idx0)
    return out


def f32_to_bf16(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().alo_f32_to_bf16_array(_ptr(out), _ptr(a), a.size)
    return out


def f32_to_f16(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().alo_f32_to_f16_array(_ptr(out), _ptr(a), a.size)
    return out


def bf16_to_f32(a):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().alo_bf16_to_f32_array(_ptr(out), _ptr(a), a.size)
    return out


def f16_to_f32(a):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().alo_f16_to_f32_array(_ptr(out), _ptr(a), a.size)
    return out


def step(inout, inn, dtype, op):
    """Returns in OP inout (a new array; the MPI user-op rule inout = in OP inout)."""
    res = np.array(inout, copy=True)
    inn = np.ascontiguousarray(inn)
    assert res.dtype == inn.dtype and res.size == inn.size
    rc = lib().alo_step(_ptr(res), _ptr(inn), res.size, _dt(dtype), _op(op))
    if rc:
        raise ValueError("Reduction operator not supported")
    return res


def divide(x, dtype, ranks):
    """Returns x / ranks (a new array): the division that ends an avg."""
    res = np.array(x, copy=True)
    rc = lib().alo_divide(_ptr(res), res.size, _dt(dtype), ranks)
    if rc:
        raise ValueError("bad divide arguments")
    return res


def schedule(P, order, start=0):
    pairs = (C.c_int * (2 * max(P, 1)))()
    result = C.c_int(0)
    n = lib().alo_schedule(P, _order(order), start, pairs, C.byref(result))
    if n < 0:
        raise ValueError("bad schedule arguments")
    return [(pairs[2 * k], pairs[2 * k + 1]) for k in range(n)], result.value


def combine(ins, dtype, op, order="rank_asc", start=0):
    ins = [np.ascontiguousarray(a) for a in ins]
    out = np.empty_like(ins[0])
    rc = lib().alo_combine(_ptr(out), _ptr_array(ins), len(ins), ins[0].size, _dt(dtype),
                           _op(op), _order(order), start)
    if rc:
        raise ValueError("Reduction operator not supported" if rc == 1 else "oracle error %d" % rc)
    return out


def combine_generated(P, n, dtype, op, order, start, dist, seed_base, idx0=0):
    out = np.empty(n, dtype=NP_CARRIER[DTYPES[_dt(dtype)]])
    rc = lib().alo_combine_generated(_ptr(out), P, n, _dt(dtype), _op(op), _order(order), start,
                                     _dist(dist), seed_base, idx0)
    if rc:
        raise ValueError("oracle error %d" % rc)
    return out


def reduce_scatter(sends, dtype, op, order):
    P = len(sends)
    sends = [np.ascontiguousarray(a) for a in sends]
    count = sends[0].size // P
    recvs = [np.empty(count, dtype=sends[0].dtype) for _ in range(P)]
    rc = lib().alo_reduce_scatter(_ptr_array(recvs), _ptr_array(sends), P, count, _dt(dtype),
                                  _op(op), _order(order))
    if rc:
        raise ValueError("oracle error %d" % rc)
    return recvs


def allgather(sends, dtype):
    P = len(sends)
    sends = [np.ascontiguousarray(a) for a in sends]
    count = sends[0].size
    recvs = [np.empty(count * P, dtype=sends[0].dtype) for _ in range(P)]
    rc = lib().alo_allgather(_ptr_array(recvs), _ptr_array(sends), P, count, _dt(dtype))
    if rc:
        raise ValueError("oracle error %d" % rc)
    return recvs


def reduce_scatterv(sends, counts, dtype, op, order):
    P = len(sends)
    sends = [np.ascontiguousarray(a) for a in sends]
    recvs = [np.empty(counts[b], dtype=sends[0].dtype) for b in range(P)]
    rc = lib().alo_reduce_scatterv(_ptr_array(recvs), _ptr_array(sends), P, (C.c_size_t * P)(*counts),
                                   _dt(dtype), _op(op), _order(order))
    if rc:
        raise ValueError("oracle error %d" % rc)
    return recvs


def allgatherv(sends, counts, displs, dtype, fill_value=0):
    """Returns the P receive buffers (positions no slice covers hold `fill_value`)."""
    P = len(sends)
    sends = [np.ascontiguousarray(a) for a in sends]
    extent = max([d + c for c, d in zip(counts, displs) if c] + [0])
    recvs = [np.full(extent, fill_value, dtype=sends[0].dtype) for _ in range(P)]
    rc = lib().alo_allgatherv(_ptr_array(recvs), _ptr_array(sends), P, (C.c_size_t * P)(*counts),
                              (C.c_size_t * P)(*displs), _dt(dtype))
    if rc:
        raise ValueError("oracle error %d" % rc)
    return recvs


def ring_segment(n, P, s):
    off, ln = C.c_size_t(0), C.c_size_t(0)
    lib().alo_ring_segment(n, P, s, C.byref(off), C.byref(ln))
    return off.value, ln.value


def ring_allreduce(bufs, dtype, op, chunk_elems):
    """In place on copies; returns the P final buffers."""
    bufs = [np.array(b, copy=True) for b in bufs]
    rc = lib().alo_ring_allreduce(_ptr_array(bufs), len(bufs), bufs[0].size, _dt(dtype), _op(op),
                                  chunk_elems)
    if rc:
        raise ValueError("oracle error %d" % rc)
    return bufs


def ring_reduce_scatter(bufs, dtype, op, chunk_elems):
    bufs = [np.array(b, copy=True) for b in bufs]
    rc = lib().alo_ring_reduce_scatter(_ptr_array(bufs), len(bufs), bufs[0].size, _dt(dtype),
                                       _op(op), chunk_elems)
    if rc:
        raise ValueError("oracle error %d" % rc)
    return bufs


def ring_allgather(bufs, dtype, chunk_elems):
    bufs = [np.array(b, copy=True) for b in bufs]
    rc = lib().alo_ring_allgather(_ptr_array(bufs), len(bufs), bufs[0].size, _dt(dtype),
                                  chunk_elems)
    if rc:
        raise ValueError("oracle error %d" % rc)
    return bufs


def halo_face_elems(nx, ny, nz, h, face):
    return lib().alo_halo_face_elems(nx, ny, nz, h, face)


def halo_pack(grid, nx, ny, nz, h, face):
    grid = np.ascontiguousarray(grid)
    buf = np.empty(halo_face_elems(nx, ny, nz, h, face), dtype=grid.dtype)
    rc = lib().alo_halo_pack(_ptr(buf), _ptr(grid), nx, ny, nz, h, face, grid.itemsize)
    if rc:
        raise ValueError("oracle error %d" % rc)
    return buf


def halo_unpack(grid, buf, nx, ny, nz, h, face):
    """Returns a copy of `grid` with the ghost slab of `face` overwritten from `buf`."""
    grid = np.array(grid, copy=True)
    buf = np.ascontiguousarray(buf)
    rc = lib().alo_halo_unpack(_ptr(grid), _ptr(buf), nx, ny, nz, h, face, grid.itemsize)
    if rc:
        raise ValueError("oracle error %d" % rc)
    return grid


def checksum(a):
    a = np.ascontiguousarray(a)
    return lib().alo_checksum(_ptr(a), a.nbytes)


def num_threads():
    return lib().alo_num_threads()


def set_num_threads(n):
    lib().alo_set_num_threads(n)
