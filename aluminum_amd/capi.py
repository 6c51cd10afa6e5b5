"""ctypes binding of the C ABI in include/aluminum_amd.h.

Tensors are torch tensors on the GPU; only their ``data_ptr()`` crosses the
boundary.  fp16 / bf16 may be passed either as torch.float16 / torch.bfloat16
tensors or as raw int16 bit patterns together with an explicit dtype name.
Work is enqueued on torch's current stream unless a stream is given.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libaluminum_amd.so")

DTYPES = ["i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64", "f16", "bf16", "f32", "f64"]
OPS = ["sum", "prod", "min", "max", "lor", "land", "lxor", "bor", "band", "bxor", "avg"]
ORDERS = {"rank_asc": 0, "tree_dbl": 1, "tree_halv": 2, "pairwise_desc": 3, "ring": 4,
          "tree_binomial": 5, "tree_rsg": 6, "tree_rsg_spread": 7}
DISTS = {"uniform_pm1": 0, "uniform_09_11": 1, "uniform_01": 2, "fullrange": 3, "bool01": 4,
         "normal": 5, "smallint": 6}
RING_MODES = {"stepwise": 0, "fused": 1}
FLAG_MODES = {"auto": 0, "memop": 1, "kernel": 2}

STATUS = {1: "invalid argument", 2: "unsupported reduction operator", 3: "unsupported type",
          4: "invalid algorithm", 5: "overlapping buffers", 6: "HIP error", 7: "timeout",
          8: "unsupported"}


class AlError(RuntimeError):
    """Mirror of Al::al_exception: raised for every nonzero status."""

    def __init__(self, code, message):
        super().__init__("%s (status %d: %s)" % (message, code, STATUS.get(code, "?")))
        self.code = code
        self.message = message


_lib = None


def lib_path():
    return _LIB


def load():
    """Loads libaluminum_amd.so; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB):
        raise ImportError("libaluminum_amd.so is not built: run `make -C aluminum_amd/csrc` "
                          "or __graft_entry__.build()")
    L = C.CDLL(_LIB)
    vp, sz, i, u64, i32 = C.c_void_p, C.c_size_t, C.c_int, C.c_uint64, C.c_int32
    pvp = C.POINTER(vp)
    L.alamd_last_error.restype = C.c_char_p
    L.alamd_version.restype = i
    L.alamd_dtype_size.restype = sz
    L.alamd_dtype_size.argtypes = [i]
    L.alamd_check_op.argtypes = [i, i]
    L.alamd_init.argtypes = []
    L.alamd_reference_order.argtypes = [i, i, sz, i, i, C.POINTER(i), C.POINTER(i)]
    L.alamd_combine.argtypes = [pvp, i, pvp, i, sz, i, i, i, i, vp]
    L.alamd_reduce_scatter.argtypes = [pvp, pvp, i, sz, i, i, i, vp]
    L.alamd_allgather.argtypes = [pvp, pvp, i, sz, i, vp]
    L.alamd_reduce_scatterv.argtypes = [pvp, pvp, i, C.POINTER(sz), i, i, i, vp]
    L.alamd_reduce_scatterv_noalloc.argtypes = [pvp, pvp, i, C.POINTER(sz), i, i, i, vp]
    L.alamd_allgatherv.argtypes = [pvp, pvp, i, C.POINTER(sz), C.POINTER(sz), i, vp]
    L.alamd_reduce_scatterv_wait_expired.argtypes = []
    L.alamd_set_chain_poll_limit.argtypes = [C.c_uint]
    L.alamd_reserve_scratch.argtypes = [vp, sz]
    L.alamd_release_scratch.argtypes = [vp]
    L.alamd_tune.argtypes = [C.c_char_p, sz]
    L.alamd_tuned.argtypes = [C.c_char_p]
    L.alamd_tuned.restype = sz
    L.alamd_planned_launches.argtypes = [i, sz, i]
    L.alamd_planned_launches.restype = sz
    L.alamd_ring_allreduce.argtypes = [pvp, i, sz, i, i, sz, i, vp]
    L.alamd_ring_allreduce_from.argtypes = [pvp, pvp, i, sz, i, i, sz, i, vp]
    L.alamd_ring_reduce_scatter.argtypes = [pvp, i, sz, i, i, sz, i, vp]
    L.alamd_ring_allgather.argtypes = [pvp, i, sz, i, sz, vp]
    L.alamd_ring_segment.argtypes = [sz, i, i, C.POINTER(sz), C.POINTER(sz)]
    L.alamd_halo_pack.argtypes = [pvp, vp, C.POINTER(sz), sz, sz, C.c_uint, vp]
    L.alamd_halo_unpack.argtypes = [vp, pvp, C.POINTER(sz), sz, sz, C.c_uint, vp]
    L.alamd_halo_face_elems.restype = sz
    L.alamd_halo_face_elems.argtypes = [C.POINTER(sz), sz, i]
    L.alamd_flag_create.argtypes = [pvp, i32]
    L.alamd_flag_destroy.argtypes = [vp]
    L.alamd_flag_host_ptr.restype = vp
    L.alamd_flag_host_ptr.argtypes = [vp]
    L.alamd_stream_memops_supported.restype = i
    L.alamd_stream_wait_flag.argtypes = [vp, vp, i32, i, u64]
    L.alamd_stream_write_flag.argtypes = [vp, vp, i32, i]
    L.alamd_flag_signal.argtypes = [vp, i32]
    L.alamd_flag_query.restype = i32
    L.alamd_flag_query.argtypes = [vp]
    L.alamd_flag_timed_out.argtypes = [vp]
    L.alamd_fill.argtypes = [vp, sz, i, i, u64, u64, vp]
    L.alamd_narrow_f32.argtypes = [vp, vp, sz, i, vp]
    L.alamd_widen_f32.argtypes = [vp, vp, sz, i, vp]
    L.alamd_copy.argtypes = [vp, vp, sz, vp]
    _lib = L
    return L


def _check(rc):
    if rc != 0:
        raise AlError(rc, load().alamd_last_error().decode())


def _dt(dtype):
    return DTYPES.index(dtype) if isinstance(dtype, str) else int(dtype)


def _op(op):
    return OPS.index(op) if isinstance(op, str) else int(op)


def _order(order):
    return ORDERS[order] if isinstance(order, str) else int(order)


def dtype_size(dtype):
    return load().alamd_dtype_size(_dt(dtype))


def check_op(dtype, op):
    _check(load().alamd_check_op(_dt(dtype), _op(op)))


def torch_dtype(dtype):
    """torch carrier dtype of a library dtype (unsigned 16/32/64 and the 16-bit
    floats are carried as the signed integer of the same width)."""
    import torch
    return {"i8": torch.int8, "u8": torch.uint8, "i16": torch.int16, "u16": torch.int16,
            "i32": torch.int32, "u32": torch.int32, "i64": torch.int64, "u64": torch.int64,
            "f16": torch.int16, "bf16": torch.int16, "f32": torch.float32,
            "f64": torch.float64}[dtype]


def _infer_dtype(t):
    import torch
    return {torch.int8: "i8", torch.uint8: "u8", torch.int16: "i16", torch.int32: "i32",
            torch.int64: "i64", torch.float16: "f16", torch.bfloat16: "bf16",
            torch.float32: "f32", torch.float64: "f64"}[t.dtype]


def _stream(stream):
    import torch
    if stream is None:
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)
    if isinstance(stream, int):
        return C.c_void_p(stream)
    return C.c_void_p(stream.cuda_stream)


def _table(tensors):
    arr = (C.c_void_p * len(tensors))()
    for k, t in enumerate(tensors):
        if t is None:
            arr[k] = None
            continue
        if not t.is_cuda:
            raise AlError(1, "buffers must live on the GPU")
        if not t.is_contiguous():
            raise AlError(1, "buffers must be contiguous")
        arr[k] = t.data_ptr()
    return arr


def combine(outs, ins, op, order="rank_asc", start=0, dtype=None, count=None, stream=None):
    """outs[j][:] = fold of ins[0..P-1] in the named order (alamd_combine)."""
    dtype = dtype or _infer_dtype(ins[0])
    count = ins[0].numel() if count is None else count
    _check(load().alamd_combine(_table(outs), len(outs), _table(ins), len(ins), count, _dt(dtype),
                                _op(op), _order(order), start, _stream(stream)))


COLLECTIVES = {"allreduce": 0, "reduce": 1, "reduce_scatter": 2, "allreduce_blocking": 3, "reduce_blocking": 4}
_ORDER_NAMES = {v: k for k, v in ORDERS.items()}


def reference_order(collective, P, count, dtype, root=0):
    """(order name, start) the reference's result follows for this collective (alamd_reference_order)."""
    order, start = C.c_int(0), C.c_int(0)
    _check(load().alamd_reference_order(COLLECTIVES[collective], P, count, _dt(dtype), root, C.byref(order),
                                        C.byref(start)))
    return _ORDER_NAMES[order.value], start.value


def reduce_scatter(recvs, sends, op, order="rank_asc", dtype=None, count=None, stream=None):
    dtype = dtype or _infer_dtype(sends[0])
    P = len(sends)
    count = sends[0].numel() // P if count is None else count
    _check(load().alamd_reduce_scatter(_table(recvs), _table(sends), P, count, _dt(dtype), _op(op),
                                       _order(order), _stream(stream)))


def allgather(recvs, sends, dtype=None, count=None, stream=None):
    dtype = dtype or _infer_dtype(sends[0])
    count = sends[0].numel() if count is None else count
    _check(load().alamd_allgather(_table(recvs), _table(sends), len(sends), count, _dt(dtype),
                                  _stream(stream)))


def reduce_scatterv(recvs, sends, counts, op, order="rank_asc", dtype=None, stream=None):
    dtype = dtype or _infer_dtype(sends[0])
    P = len(sends)
    _check(load().alamd_reduce_scatterv(_table(recvs), _table(sends), P, (C.c_size_t * P)(*counts), _dt(dtype),
                                        _op(op), _order(order), _stream(stream)))


def reduce_scatterv_noalloc(recvs, sends, counts, op, order="rank_asc", dtype=None, stream=None):
    """alamd_reduce_scatterv_noalloc: the same call with its scratch in a fixed device array."""
    dtype = dtype or _infer_dtype(sends[0])
    P = len(sends)
    _check(load().alamd_reduce_scatterv_noalloc(_table(recvs), _table(sends), P, (C.c_size_t * P)(*counts),
                                                _dt(dtype), _op(op), _order(order), _stream(stream)))


def reduce_scatterv_wait_expired():
    """True, once, if a wait inside a chained in-place Reduce_scatterv launch has given up since the last call."""
    return bool(load().alamd_reduce_scatterv_wait_expired())


CHAIN_POLLS_NONE = 0xffffffff  # every wait the tiling calls for gives up without looking


def set_chain_poll_limit(polls):
    """Polls after which such a wait gives up (0: the default; CHAIN_POLLS_NONE); for tests of that path."""
    _check(load().alamd_set_chain_poll_limit(polls))


def reserve_scratch(max_block_bytes, stream=None):
    """alamd_reserve_scratch: scratch for in-place Reduce_scatterv blocks of up to that many bytes on `stream`."""
    _check(load().alamd_reserve_scratch(_stream(stream), max_block_bytes))


def release_scratch(stream=None):
    _check(load().alamd_release_scratch(_stream(stream)))


def tune(name, value):
    """Sets one of the launch planners' sizes (0: its default); speed only, never results."""
    _check(load().alamd_tune(name.encode(), value))


def tuned(name):
    return int(load().alamd_tuned(name.encode()))


def planned_launches(P, count, dtype):
    """Kernel launches of one alamd_combine call with one output (alamd_planned_launches)."""
    return int(load().alamd_planned_launches(P, count, _dt(dtype)))


def allgatherv(recvs, sends, counts, displs, dtype=None, stream=None):
    dtype = dtype or _infer_dtype(recvs[0])
    P = len(recvs)
    _check(load().alamd_allgatherv(_table(recvs), _table(sends), P, (C.c_size_t * P)(*counts),
                                   (C.c_size_t * P)(*displs), _dt(dtype), _stream(stream)))


def ring_allreduce(bufs, op, chunk_bytes=4 << 20, mode="stepwise", dtype=None, count=None,
                   stream=None, sends=None):
    """In place on bufs, or (sends given) from sends into bufs."""
    dtype = dtype or _infer_dtype(bufs[0])
    count = bufs[0].numel() if count is None else count
    if sends is not None:
        _check(load().alamd_ring_allreduce_from(_table(bufs), _table(sends), len(bufs), count, _dt(dtype), _op(op),
                                                chunk_bytes, RING_MODES[mode], _stream(stream)))
        return
    _check(load().alamd_ring_allreduce(_table(bufs), len(bufs), count, _dt(dtype), _op(op),
                                       chunk_bytes, RING_MODES[mode], _stream(stream)))


def ring_reduce_scatter(bufs, op, chunk_bytes=4 << 20, mode="stepwise", dtype=None, count=None,
                        stream=None):
    dtype = dtype or _infer_dtype(bufs[0])
    count = bufs[0].numel() if count is None else count
    _check(load().alamd_ring_reduce_scatter(_table(bufs), len(bufs), count, _dt(dtype), _op(op),
                                            chunk_bytes, RING_MODES[mode], _stream(stream)))


def ring_allgather(bufs, chunk_bytes=4 << 20, dtype=None, count=None, stream=None):
    dtype = dtype or _infer_dtype(bufs[0])
    count = bufs[0].numel() if count is None else count
    _check(load().alamd_ring_allgather(_table(bufs), len(bufs), count, _dt(dtype), chunk_bytes,
                                       _stream(stream)))


def ring_segment(count, P, s):
    off, ln = C.c_size_t(0), C.c_size_t(0)
    _check(load().alamd_ring_segment(count, P, s, C.byref(off), C.byref(ln)))
    return off.value, ln.value


def _dims(dims):
    return (C.c_size_t * 3)(*dims)


def halo_face_elems(dims, halo, face):
    return load().alamd_halo_face_elems(_dims(dims), halo, face)


def _face_table(bufs):
    tab = [None] * 6
    mask = 0
    for f, t in bufs.items():
        tab[f] = t
        mask |= 1 << f
    return _table(tab), mask


def halo_pack(bufs, grid, dims, halo, stream=None):
    """bufs: {face: tensor}.  dims = interior (nx, ny, nz), x fastest."""
    tab, mask = _face_table(bufs)
    _check(load().alamd_halo_pack(tab, C.c_void_p(grid.data_ptr()), _dims(dims), halo,
                                  grid.element_size(), mask, _stream(stream)))


def halo_unpack(grid, bufs, dims, halo, stream=None):
    tab, mask = _face_table(bufs)
    _check(load().alamd_halo_unpack(C.c_void_p(grid.data_ptr()), tab, _dims(dims), halo,
                                    grid.element_size(), mask, _stream(stream)))


def fill(t, dist, seed, idx0=0, dtype=None, count=None, stream=None):
    dtype = dtype or _infer_dtype(t)
    count = t.numel() if count is None else count
    _check(load().alamd_fill(C.c_void_p(t.data_ptr()), count, _dt(dtype), DISTS[dist], seed, idx0,
                             _stream(stream)))


def narrow_f32(dst16, src, dtype, stream=None):
    _check(load().alamd_narrow_f32(C.c_void_p(dst16.data_ptr()), C.c_void_p(src.data_ptr()),
                                   src.numel(), _dt(dtype), _stream(stream)))


def widen_f32(dst, src16, dtype, stream=None):
    _check(load().alamd_widen_f32(C.c_void_p(dst.data_ptr()), C.c_void_p(src16.data_ptr()),
                                  src16.numel(), _dt(dtype), _stream(stream)))


def copy(dst, src, nbytes=None, stream=None):
    nbytes = src.numel() * src.element_size() if nbytes is None else nbytes
    _check(load().alamd_copy(C.c_void_p(dst.data_ptr()), C.c_void_p(src.data_ptr()), nbytes,
                             _stream(stream)))


class Flag:
    """One synchronisation word (alamd_flag)."""

    def __init__(self, initial=0):
        self._h = C.c_void_p(None)
        _check(load().alamd_flag_create(C.byref(self._h), initial))

    def wait(self, value=1, mode="auto", max_spins=0, stream=None):
        _check(load().alamd_stream_wait_flag(_stream(stream), self._h, value, FLAG_MODES[mode],
                                             max_spins))

    def write(self, value=1, mode="auto", stream=None):
        _check(load().alamd_stream_write_flag(_stream(stream), self._h, value, FLAG_MODES[mode]))

    def signal(self, value=1):
        _check(load().alamd_flag_signal(self._h, value))

    def query(self):
        return load().alamd_flag_query(self._h)

    def timed_out(self):
        return bool(load().alamd_flag_timed_out(self._h))

    def destroy(self):
        if self._h:
            _check(load().alamd_flag_destroy(self._h))
            self._h = C.c_void_p(None)


def memops_supported():
    return bool(load().alamd_stream_memops_supported())
