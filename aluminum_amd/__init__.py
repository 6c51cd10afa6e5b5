"""aluminum_amd: MI355X on-device combine engine behind Aluminum's
Al::Allreduce / Reduce_scatter / Allgather (C-ABI library + thin bindings).

The product is ``libaluminum_amd.so`` (HIP kernels and the C ABI declared in
``include/aluminum_amd.h``) and the header-only C++ shim
``include/aluminum_amd/Al.hpp``.  This Python package only binds the C ABI
with ctypes so that tests and the benchmark can drive it with torch tensors as
device memory.  There is no CPU fallback: if the library is missing or no GPU
is present, calls raise.
"""
from . import capi  # noqa: F401
from .capi import (  # noqa: F401
    AlError, DTYPES, OPS, ORDERS, DISTS, RING_MODES, FLAG_MODES,
    load, lib_path, combine, reduce_scatter, allgather, reduce_scatterv, reduce_scatterv_noalloc, allgatherv,
    reduce_scatterv_wait_expired, set_chain_poll_limit, tune, tuned, reference_order, reserve_scratch,
    release_scratch, CHAIN_POLLS_NONE, planned_launches,
    ring_allreduce,
    ring_reduce_scatter, ring_allgather, halo_pack, halo_unpack, halo_face_elems,
    fill, narrow_f32, widen_f32, copy, Flag, torch_dtype, dtype_size, check_op,
)
