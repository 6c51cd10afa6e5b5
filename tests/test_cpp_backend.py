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
    bad = subprocess.run([exe, "--op", "allreduce", "--reduction-op", "avg", "--max-size", "4"], capture_output=True,
                         text=True, timeout=60)
    assert bad.returncode == 1 and "Reduction operator not supported" in bad.stderr
