"""The C-ABI library: it loads, exports every symbol the header declares, and
its host-side argument checks answer before any GPU work is attempted."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "aluminum_amd.h")


SUPPORT_HEADER = os.path.join(ROOT, "include", "aluminum_amd_support.h")


def declared_functions():
    text = open(HEADER).read() + open(SUPPORT_HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(alamd_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ("alamd_combine", "alamd_reduce_scatter", "alamd_allgather", "alamd_ring_allreduce",
                 "alamd_halo_pack", "alamd_halo_unpack", "alamd_stream_wait_flag", "alamd_stream_write_flag",
                 "alamd_flag_signal", "alamd_flag_query", "alamd_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    import aluminum_amd
    lib = aluminum_amd.load()
    for name in declared_functions():
        assert hasattr(lib, name), "libaluminum_amd.so does not export %s" % name


def test_enums_match_the_reference_numbering():
    # include/aluminum/base.hpp:103-105
    text = open(HEADER).read()
    for k, name in enumerate(["SUM", "PROD", "MIN", "MAX", "LOR", "LAND", "LXOR", "BOR", "BAND", "BXOR", "AVG"]):
        assert re.search(r"ALAMD_%s = %d\b" % (name, k), text), name
    ref = "/root/reference/include/aluminum/base.hpp"
    if os.path.exists(ref):
        m = re.search(r"enum class ReductionOperator \{([^}]*)\}", open(ref).read(), flags=re.S)
        assert [s.strip() for s in m.group(1).split(",")] == ["sum", "prod", "min", "max", "lor", "land", "lxor",
                                                               "bor", "band", "bxor", "avg"]


def test_dtype_table_and_op_support():
    import aluminum_amd as al
    sizes = dict(i8=1, u8=1, i16=2, u16=2, i32=4, u32=4, i64=8, u64=8, f16=2, bf16=2, f32=4, f64=8)
    for k, v in sizes.items():
        assert al.dtype_size(k) == v
    assert al.load().alamd_dtype_size(99) == 0
    import oracle
    for dt in al.DTYPES:
        for op in al.OPS:
            ok = al.load().alamd_check_op(al.DTYPES.index(dt), al.OPS.index(op)) == 0
            assert ok == (oracle.check_op(dt, op) == 0), (dt, op)


def test_argument_checks_need_no_gpu():
    import aluminum_amd as al
    L = al.load()
    one = (C.c_void_p * 1)(0x1000)
    two = (C.c_void_p * 2)(0x2000, 0x3000)
    f32, SUM, AVG = al.DTYPES.index("f32"), 0, 10
    assert L.alamd_combine(one, 1, two, 0, 16, f32, SUM, 0, 0, None) == 1          # P = 0
    assert L.alamd_combine(one, 1, two, 65, 16, f32, SUM, 0, 0, None) == 1         # P too large
    assert L.alamd_combine(one, 1, two, 2, 16, f32, AVG + 1, 0, 0, None) == 2
    assert b"Reduction operator not supported" in L.alamd_last_error()
    assert L.alamd_combine(one, 1, two, 2, 16, f32, 7, 0, 0, None) == 2            # bor on fp32
    assert L.alamd_combine(one, 1, two, 2, 16, 42, SUM, 0, 0, None) == 3
    assert L.alamd_combine(one, 1, two, 2, 16, f32, SUM, 9, 0, None) == 4
    assert b"Invalid algorithm" in L.alamd_last_error()
    assert L.alamd_combine(one, 1, two, 2, 16, f32, SUM, 0, 1, None) == 1          # start without an order that has one
    assert L.alamd_combine(one, 1, two, 2, 16, f32, SUM, 4, 2, None) == 1          # start out of range
    over = (C.c_void_p * 1)(0x2010)
    assert L.alamd_combine(over, 1, two, 2, 16, f32, SUM, 0, 0, None) == 5         # partial overlap
    assert L.alamd_combine(one, 1, two, 2, 0, f32, SUM, 0, 0, None) == 0           # empty: nothing to do
    assert L.alamd_reduce_scatter(two, two, 2, 0, f32, SUM, 0, None) == 0
    assert L.alamd_allgather(two, two, 2, 0, f32, None) == 0
    assert L.alamd_ring_allreduce(two, 2, 16, f32, SUM, 6, 0, None) == 1           # chunk not a multiple of 4
    assert L.alamd_ring_allreduce(two, 2, 16, f32, SUM, 64, 5, None) == 4          # unknown mode
    assert L.alamd_ring_allreduce(two, 2, 0, f32, SUM, 64, 0, None) == 0
    off, ln = C.c_size_t(), C.c_size_t()
    assert L.alamd_ring_segment(10, 4, 1, C.byref(off), C.byref(ln)) == 0 and (off.value, ln.value) == (3, 3)
    assert L.alamd_ring_segment(10, 4, 3, C.byref(off), C.byref(ln)) == 0 and (off.value, ln.value) == (8, 2)
    dims = (C.c_size_t * 3)(8, 8, 8)
    assert L.alamd_halo_face_elems(dims, 2, 0) == 2 * 8 * 8
    assert L.alamd_halo_face_elems(dims, 2, 6) == 0
    six = (C.c_void_p * 6)(*([0x9000] * 6))
    assert L.alamd_halo_pack(six, 0x1000, dims, 9, 8, 0x3f, None) == 1             # halo wider than interior
    assert L.alamd_halo_pack(six, 0x1000, dims, 2, 3, 0x3f, None) == 3             # odd element size
    assert L.alamd_halo_pack(six, 0x1000, dims, 2, 8, 0x40, None) == 1             # face 6
    assert L.alamd_halo_pack(six, 0x1000, dims, 2, 8, 0, None) == 0                # no face selected
    assert L.alamd_fill(0x1000, 16, 42, 0, 1, 0, None) == 3
    assert L.alamd_fill(0x1000, 16, f32, 42, 1, 0, None) == 1
    assert L.alamd_version() >= 1


def test_launch_planner_sizes_are_checked():
    """alamd_tune: unknown names and piece sizes that would never finish a call are errors; 0 restores a default."""
    import aluminum_amd as al
    default = al.tuned("ring_piece_bytes")
    assert default == 256 << 20 and al.tuned("no such size") == 0
    al.tune("ring_piece_bytes", 1 << 20)
    assert al.tuned("ring_piece_bytes") == 1 << 20
    al.tune("ring_piece_bytes", 0)
    assert al.tuned("ring_piece_bytes") == default
    for name, value in (("two_step_piece_bytes", 4), ("ring_piece_bytes", 1000), ("no such size", 1 << 20)):
        with pytest.raises(al.AlError):
            al.tune(name, value)
    assert al.tuned("two_step_piece_bytes") == 128 << 20


def test_planned_launches_follow_the_launch_cut_and_the_shape():
    """alamd_planned_launches runs the fold's planner without launching: one launch up to 4 GiB of traffic,
    then a power of two of tiles per launch; a call of middling size counts in the 16 KiB tiles of the
    block shape, the others in the 1 KiB tiles of the streaming shape."""
    import aluminum_amd as al
    assert al.tuned("launch_bytes") == 4 << 30
    assert al.tuned("block_shape_from_bytes") == 32 << 20 and al.tuned("block_shape_below_bytes") == 384 << 20
    assert al.planned_launches(8, 1 << 26, "f32") == 1      # the headline workload: 9 x 256 MiB
    assert al.planned_launches(8, 1 << 28, "f32") == 4      # 9 GiB: 256 MiB per stream and launch
    assert al.planned_launches(64, 1 << 28, "f32") == 32    # 65 GiB: 32 MiB per stream and launch
    assert al.planned_launches(8, 1 << 22, "f32") == 1      # 144 MiB in all: block shape
    assert al.planned_launches(8, 0, "f32") == 0
    try:
        al.tune("launch_bytes", 9 << 20)  # 1 MiB per stream and launch at P = 8, whatever the tile
        assert al.planned_launches(8, 1 << 26, "f32") == 256
        assert al.planned_launches(8, 1 << 22, "f32") == 16
        al.tune("launch_bytes", 1)        # never fewer than eight tiles per launch: 8 KiB streaming, 128 KiB in blocks
        assert al.planned_launches(8, 1 << 20, "f32") == 32    # 36 MiB in all: block shape
        assert al.planned_launches(8, 1 << 18, "f32") == 128   # 9 MiB in all: streaming
    finally:
        al.tune("launch_bytes", 0)
    assert al.tuned("launch_bytes") == 4 << 30


def test_graft_entry_has_build_and_smoke():
    import importlib
    g = importlib.import_module("__graft_entry__")
    assert callable(g.build) and callable(g.smoke)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True)
    assert p.returncode != 0 and "one GPU" in p.stderr
