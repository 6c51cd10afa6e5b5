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
