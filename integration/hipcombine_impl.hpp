// Al::HipCombineBackend as one more backend of Aluminum itself.
//
// A maintainer includes this header at the end of the reference's include/Al.hpp, next to the other
// backends (include/Al.hpp:2005-2014), behind a configuration macro of their choice, with this
// repository's include/ directory on the include path and libaluminum_amd.so on the link line.
// Everything before that point in Al.hpp stays as it is: Al::ReductionOperator, Al::al_exception,
// Al::AlOperation, the trait templates (include/aluminum/traits/traits_base.hpp) and the
// Al::Allreduce / Reduce / Reduce_scatter(v) / Allgather(v) / Test / Wait templates are the
// reference's own; this header adds the backend class they are instantiated with, its trait
// specialisations (what include/aluminum/traits/ht_traits.hpp is for the host-transfer backend) and
// its Test / Wait specialisations (include/aluminum/ht_impl.hpp:1113-1138).
//
// The backend's communicator is Al::amd::Communicator: P logical ranks of one GPU held by an
// Al::amd::World, each with a stream, instead of an MPI communicator.
#pragma once

#define AL_AMD_WITH_REFERENCE
#include "aluminum_amd/Al.hpp"
