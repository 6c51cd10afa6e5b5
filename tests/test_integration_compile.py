"""Al::HipCombineBackend compiled as a backend of the reference itself.

One translation unit includes the reference's own include/Al.hpp, then integration/hipcombine_impl.hpp
(this repository's front end with AL_AMD_WITH_REFERENCE defined), and calls the reference's
Al::Allreduce / Reduce / Reduce_scatter(v) / Allgather(v) / Test / Wait templates (include/Al.hpp:118-207,
222-314, 329-421, 550-633) with the backend; the traits are the reference's templates
(include/aluminum/traits/traits_base.hpp:43-62, 86-92, 155-184).  The compiler is run with
-fsyntax-only: nothing is linked, nothing of the reference is built or copied.  The two headers that the
reference's configuration step writes (Al_config.hpp, aluminum/tuning_params.hpp) are written into a
temporary directory from the reference's own templates, every optional feature off.

Skipped where the reference tree, an MPI header or the HIP headers are absent (the GPU box)."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
MPI_INC = "/opt/conda/include"
HIP_INC = "/opt/rocm/include"

pytestmark = pytest.mark.skipif(
    not (os.path.exists(os.path.join(REF, "include", "Al.hpp")) and os.path.exists(os.path.join(MPI_INC, "mpi.h"))
         and os.path.exists(os.path.join(HIP_INC, "hip", "hip_runtime_api.h"))),
    reason="needs the reference tree, mpi.h and the HIP headers")

TU = r"""
#include <Al.hpp>
#include <aluminum/traits/traits.hpp>
#include "hipcombine_impl.hpp"

using B = Al::HipCombineBackend;
using Op = Al::ReductionOperator;

// numbering shared with the C ABI (include/aluminum/base.hpp:103-105)
static_assert(static_cast<int>(Op::sum) == ALAMD_SUM && static_cast<int>(Op::bxor) == ALAMD_BXOR &&
              static_cast<int>(Op::avg) == ALAMD_AVG, "ReductionOperator");
// the reference's trait templates, answered for the backend
static_assert(Al::IsOpSupported<Al::AlOperation::allreduce, B>::value && Al::IsOpSupported<Al::AlOperation::reduce, B>::value &&
              Al::IsOpSupported<Al::AlOperation::reduce_scatter, B>::value && Al::IsOpSupported<Al::AlOperation::reduce_scatterv, B>::value &&
              Al::IsOpSupported<Al::AlOperation::allgather, B>::value && Al::IsOpSupported<Al::AlOperation::allgatherv, B>::value, "collectives");
static_assert(!Al::IsOpSupported<Al::AlOperation::bcast, B>::value && !Al::IsOpSupported<Al::AlOperation::send, B>::value, "not on the path");
static_assert(Al::IsTypeSupported<B, float>::value && Al::IsTypeSupported<B, long long>::value && !Al::IsTypeSupported<B, long double>::value, "types");
static_assert(Al::IsReductionOpSupported<B, Op::sum>::value && Al::IsReductionOpSupported<B, Op::lxor>::value, "operators");
static_assert(std::is_same<Al::OpAlgoType<Al::AlOperation::allreduce, B>::type, B::allreduce_algo_type>::value, "algo type");
static_assert(std::is_same<Al::OpAlgoType<Al::AlOperation::reduce_scatterv, B>::type, B::reduce_scatterv_algo_type>::value, "algo type");
// the other backends' answers are untouched
static_assert(Al::IsOpSupported<Al::AlOperation::bcast, Al::MPIBackend>::value, "MPI backend");

template <typename T> void all_forms(Al::amd::World &w, T *a, T *b, size_t n) {
  auto &c = w.comm(0);
  const T *ca = a;
  B::req_type req = B::null_req;
  const std::vector<size_t> counts(static_cast<size_t>(c.size()), n), displs(static_cast<size_t>(c.size()), 0);
  Al::Allreduce<B>(ca, b, n, Op::sum, c);
  Al::Allreduce<B>(a, n, Op::max, c, B::allreduce_algo_type::automatic);
  Al::NonblockingAllreduce<B>(ca, b, n, Op::sum, c, req);
  Al::NonblockingAllreduce<B>(a, n, Op::sum, c, req);
  Al::Reduce<B>(ca, b, n, Op::prod, 0, c);
  Al::Reduce<B>(a, n, Op::min, 0, c);
  Al::NonblockingReduce<B>(ca, b, n, Op::sum, 0, c, req);
  Al::NonblockingReduce<B>(a, n, Op::sum, 0, c, req);
  Al::Reduce_scatter<B>(ca, b, n, Op::sum, c);
  Al::Reduce_scatter<B>(a, n, Op::sum, c);
  Al::NonblockingReduce_scatter<B>(ca, b, n, Op::sum, c, req);
  Al::NonblockingReduce_scatter<B>(a, n, Op::sum, c, req);
  Al::Reduce_scatterv<B>(ca, b, counts, Op::sum, c);
  Al::Reduce_scatterv<B>(a, counts, Op::sum, c);
  Al::NonblockingReduce_scatterv<B>(ca, b, counts, Op::sum, c, req);
  Al::NonblockingReduce_scatterv<B>(a, counts, Op::sum, c, req);
  Al::Allgather<B>(ca, b, n, c);
  Al::Allgather<B>(a, n, c);
  Al::NonblockingAllgather<B>(ca, b, n, c, req);
  Al::NonblockingAllgather<B>(a, n, c, req);
  Al::Allgatherv<B>(ca, b, counts, displs, c);
  Al::Allgatherv<B>(a, counts, displs, c);
  Al::NonblockingAllgatherv<B>(ca, b, counts, displs, c, req);
  Al::NonblockingAllgatherv<B>(a, counts, displs, c, req);
  if (!Al::Test<B>(req)) Al::Wait<B>(req);
}
template void all_forms<float>(Al::amd::World &, float *, float *, size_t);
template void all_forms<double>(Al::amd::World &, double *, double *, size_t);
template void all_forms<int>(Al::amd::World &, int *, int *, size_t);
template void all_forms<unsigned char>(Al::amd::World &, unsigned char *, unsigned char *, size_t);
"""


def configured(template, out):
    """What the reference's configuration step writes for this template with every option off."""
    defaults = {"AL_PE_NUM_CONCURRENT_OPS": "4", "AL_PE_NUM_STREAMS": "64", "AL_PE_NUM_PIPELINE_STAGES": "2",
                "AL_PE_INPUT_QUEUE_SIZE": "8192", "AL_SYNC_MEM_PREALLOC": "1024", "AL_CACHE_LINE_SIZE": "64",
                "AL_DESTRUCTIVE_INTERFERENCE_SIZE": "128"}
    with open(template) as f:
        text = f.read()
    text = re.sub(r"#cmakedefine (\w+)", r"/* #undef \1 */", text)
    text = re.sub(r"@(\w+)@", lambda m: defaults.get(m.group(1), "0"), text)
    os.makedirs(os.path.dirname(out), exist_ok=True)
    with open(out, "w") as f:
        f.write(text)


def test_backend_compiles_inside_the_reference(tmp_path):
    configured(os.path.join(REF, "cmake", "Al_config.hpp.in"), str(tmp_path / "Al_config.hpp"))
    configured(os.path.join(REF, "cmake", "tuning_params.hpp.in"), str(tmp_path / "aluminum" / "tuning_params.hpp"))
    tu = tmp_path / "tu.cpp"
    tu.write_text(TU)
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(REF, "include"),
           "-I" + str(tmp_path), "-I" + MPI_INC, "-I" + HIP_INC, "-I" + os.path.join(ROOT, "include"),
           "-I" + os.path.join(ROOT, "integration"), str(tu)]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-4000:]


def test_standalone_and_embedded_modes_differ_only_in_what_they_define(tmp_path):
    """On its own the same header still compiles and brings the definitions itself."""
    tu = tmp_path / "alone.cpp"
    tu.write_text('#include "aluminum_amd/Al.hpp"\n'
                  "static_assert(static_cast<int>(Al::ReductionOperator::avg) == ALAMD_AVG, \"\");\n"
                  "static_assert(Al::IsOpSupported<Al::AlOperation::allreduce, Al::HipCombineBackend>::value, \"\");\n")
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I" + HIP_INC,
           "-I" + os.path.join(ROOT, "include"), str(tu)]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-4000:]
