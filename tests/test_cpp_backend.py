"""The Aluminum-shaped C++ front end (include/aluminum_amd/Al.hpp): it compiles
as plain host C++ on the CPU, and its parity program passes on the GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "test_backend")


def test_front_end_compiles_with_the_host_compiler():
    import aluminum_amd
    import oracle
    aluminum_amd.load()
    oracle.lib()
    subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"), "-B"], check=True,
                   stdout=subprocess.DEVNULL)
    assert os.path.exists(EXE)


def test_launch_planner_covers_every_tile_once():
    """plan_launches (alamd_dispatch.h) on random segment tables, on the host: every tile of every
    segment in exactly one launch, grids within the device's limits; the block lookup of the role masks
    (through prepared reciprocals) against 64-bit division and against the definition of the blocks;
    the LDS sizing of the streaming launches; the leading elements of a segment; the runs of tiles per XCD;
    which launches take the block shape."""
    exe = os.path.join(ROOT, "tests", "cpp", "test_planner")
    if not os.path.exists(exe):
        subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"), "test_planner"], check=True,
                       stdout=subprocess.DEVNULL)
    p = subprocess.run([exe, "1200"], capture_output=True, text=True, timeout=280)
    assert p.returncode == 0 and "PASSED" in p.stdout, p.stdout[-2000:] + p.stderr[-1000:]


def test_front_end_names_the_reference_interface():
    text = open(os.path.join(ROOT, "include", "aluminum_amd", "Al.hpp")).read()
    for name in ("comm_type", "req_type", "null_req", "allreduce_algo_type", "reduce_scatter_algo_type",
                 "allgather_algo_type", "NonblockingAllreduce", "Reduce_scatter", "Allgather", "RegisterMemory",
                 "static std::string Name()", "bool Test<HipCombineBackend>", "void Wait<HipCombineBackend>",
                 "local_rank", "get_stream"):
        assert name in text, name


@pytest.mark.gpu
def test_front_end_parity_program():
    assert os.path.exists(EXE), "tests/cpp/test_backend is not built (make -C tests/cpp)"
    p = subprocess.run([EXE], capture_output=True, text=True, timeout=280)
    print(p.stdout[-3000:])
    print(p.stderr[-2000:])
    assert p.returncode == 0, p.stdout[-3000:]
    assert "PASSED" in p.stdout


@pytest.mark.gpu
def test_benchmark_sweep_rows():
    """bench_ops prints the reference's per-trial rows (benchmark/benchmark_utils.hpp:151-184)."""
    exe = os.path.join(ROOT, "tests", "cpp", "bench_ops")
    assert os.path.exists(exe), "tests/cpp/bench_ops is not built (make -C tests/cpp)"
    p = subprocess.run([exe, "--op", "allreduce", "--datatype", "float", "--ranks", "4", "--max-size", "4096",
                        "--num-iters", "3", "--num-warmup", "1", "--nonblocking"], capture_output=True, text=True,
                       timeout=120)
    assert p.returncode == 0, p.stderr
    lines = p.stdout.strip().splitlines()
    assert lines[0] == "Backend Type Operation Algo NonBlocking InPlace Root CommSize Size CommRank Time"
    rows = [l.split() for l in lines[1:]]
    assert len(rows) == 13 * 4 * 3  # sizes 1..4096, 4 ranks, 3 timed trials
    for r in rows:
        assert r[0] == "HipCombineBackend" and r[2] == "allreduce" and r[4] == "1" and r[7] == "4"
        assert 0 < float(r[10]) < 1.0
    bad = subprocess.run([exe, "--op", "allreduce", "--reduction-op", "bxor", "--max-size", "4"], capture_output=True,
                         text=True, timeout=60)
    assert bad.returncode == 1 and "Reduction operator not supported" in bad.stderr
    # the summary and the file output of the reference's benchmark (benchmark/benchmark_ops.cpp:211-230)
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        out = os.path.join(d, "rows.txt")
        q = subprocess.run([exe, "--backend", "hip", "--op", "reduce_scatter", "--algorithm", "pairwise", "--ranks", "3",
                            "--size", "1000", "--num-iters", "5", "--num-warmup", "1", "--summarize", "--save-to-file",
                            out, "--no-print-table"], capture_output=True, text=True, timeout=120)
        assert q.returncode == 0, q.stderr
        shown = q.stdout.strip().splitlines()
        assert shown[0].split() == ["Size", "Mean", "Median", "Stdev", "Min", "Max"] and len(shown) == 2
        size, mean, median, stdev, lo, hi = shown[1].split()
        assert size == "1000" and 0 < float(lo) <= float(median) <= float(hi) and float(stdev) >= 0
        saved = open(out).read().strip().splitlines()
        assert saved[0] == lines[0] and len(saved) == 1 + 3 * 5
        assert all(r.split()[3] == "pairwise" and r.split()[8] == "1000" for r in saved[1:])


OPS_EXE = os.path.join(ROOT, "tests", "cpp", "test_ops")

# (arguments) in the manner of the reference's sweep (test/run_tests.py): collective x datatype x
# in place x non-blocking over power-of-two and odd sizes
OPS_SWEEPS = [
    "--op allreduce --datatype float --odd-sizes --max-size 262144 --ranks 4",
    "--op allreduce --datatype bfloat16 --inplace --nonblocking --odd-sizes --max-size 65536 --ranks 8",
    "--op allreduce --datatype half --reduction-op max --algorithm rank_order --odd-sizes --max-size 65536 --ranks 3",
    "--op allreduce --datatype uchar --reduction-op lxor --inplace --odd-sizes --max-size 65536 --ranks 5",
    "--op allreduce --datatype longlong --reduction-op band --nonblocking --max-size 65536 --ranks 8",
    "--op allreduce --datatype double --reduction-op prod --algorithm ring --min-size 0 --max-size 32768 --ranks 8",
    # more than 32 logical ranks: the default algorithm is a tree order there too
    "--op allreduce --datatype float --odd-sizes --max-size 16384 --ranks 33",
    "--op allreduce --datatype bfloat16 --inplace --max-size 16384 --ranks 64",
    "--op reduce --datatype double --root 40 --algorithm tree_binomial --max-size 4096 --ranks 48",
    "--op reduce_scatter --datatype float --max-size 256 --ranks 40",
    "--op allreduce --datatype float --reduction-op avg --inplace --odd-sizes --max-size 65536 --ranks 6",
    "--op allreduce --datatype bfloat16 --reduction-op avg --algorithm ring --max-size 32768 --ranks 8",
    "--op reduce_scatter --datatype int --reduction-op avg --nonblocking --odd-sizes --max-size 16384 --ranks 7",
    "--op reduce --datatype float --root 2 --inplace --odd-sizes --max-size 65536 --ranks 4",
    "--op reduce --datatype int --reduction-op min --root 0 --nonblocking --max-size 65536 --ranks 7",
    "--op reduce_scatter --datatype float --inplace --nonblocking --odd-sizes --max-size 65536 --ranks 8",
    "--op reduce_scatter --datatype ushort --reduction-op bor --algorithm pairwise --max-size 16384 --ranks 5",
    "--op allgather --datatype short --inplace --nonblocking --odd-sizes --max-size 65536 --ranks 8",
    "--op reduce_scatterv --datatype double --nonblocking --odd-sizes --max-size 16384 --ranks 5",
    "--op allgatherv --datatype char --inplace --nonblocking --odd-sizes --max-size 16384 --ranks 8",
    # the orders of a rooted reduce: binomial to the root (automatic below 2 KiB and for 16-bit floats),
    # reduce-scatter + gather above
    "--op reduce --datatype bfloat16 --root 6 --odd-sizes --max-size 65536 --ranks 7",
    "--op reduce --datatype float --reduction-op max --root 3 --algorithm tree_reduce_scatter_gather --odd-sizes --max-size 65536 --ranks 5",
    "--op allreduce --datatype double --reduction-op min --algorithm tree_reduce_scatter_gather --inplace --max-size 65536 --ranks 7",
    "--op reduce_scatter --datatype float --reduction-op min --algorithm tree_halving --odd-sizes --max-size 16384 --ranks 6",
    "--op allreduce --datatype float --reduction-op min --algorithm tree_reduce_scatter_gather_spread --odd-sizes --max-size 65536 --ranks 6",
    "--op reduce --datatype double --root 2 --algorithm automatic_mpi_blocking --odd-sizes --max-size 65536 --ranks 12",
    # non-blocking operations that move more than 256 MiB in all take the internal stream
    "--op allreduce --datatype double --nonblocking --odd-sizes --min-size 1048576 --max-size 4194304 --ranks 8",
    "--op reduce_scatter --datatype float --nonblocking --inplace --min-size 1048576 --max-size 2097152 --ranks 8",
    # several threads at once, each with communicators and a stream of its own (test/test_ops.cpp:373-391)
    "--op allreduce --datatype float --threads 4 --odd-sizes --max-size 262144 --ranks 4",
    "--op allreduce --datatype bfloat16 --threads 3 --nonblocking --algorithm ring --max-size 65536 --ranks 8",
    "--op reduce_scatterv --datatype float --threads 4 --inplace --odd-sizes --max-size 1048576 --ranks 8",
    "--op allgatherv --datatype int --threads 4 --nonblocking --odd-sizes --max-size 65536 --ranks 5",
    "--op allreduce --datatype double --threads 2 --nonblocking --min-size 2097152 --max-size 4194304 --ranks 8",
]


@pytest.mark.gpu
@pytest.mark.parametrize("args", OPS_SWEEPS)
def test_ops_sweep(args):
    assert os.path.exists(OPS_EXE), "tests/cpp/test_ops is not built (make -C tests/cpp)"
    p = subprocess.run([OPS_EXE] + args.split(), capture_output=True, text=True, timeout=280)
    print(p.stdout[-3000:])
    print(p.stderr[-2000:])
    assert p.returncode == 0, p.stdout[-3000:]
    assert "PASSED" in p.stdout


def test_ops_rejects_bad_arguments():
    """Argument errors are reported before any GPU call."""
    if not os.path.exists(OPS_EXE):
        pytest.skip("tests/cpp/test_ops is not built")
    for args in ("--op alltoall", "--op allreduce --backend nccl", "--op allreduce --reduction-op median",
                 "--op allreduce --ranks 4 --root 9", "--op allreduce --bogus"):
        p = subprocess.run([OPS_EXE] + args.split(), capture_output=True, text=True, timeout=60)
        assert p.returncode == 2, (args, p.stdout, p.stderr)
