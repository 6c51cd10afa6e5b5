// Fold kernels of the 32- and 64-bit integer types.
#include "combine_fold_impl.h"

namespace alamd {
namespace {
ALAMD_FOLD_GROUP(group, case ALAMD_I32: return dispatch_int_op<int32_t>(op, run);
                 case ALAMD_U32: return dispatch_int_op<uint32_t>(op, run);
                 case ALAMD_I64: return dispatch_int_op<int64_t>(op, run);
                 case ALAMD_U64: return dispatch_int_op<uint64_t>(op, run);)
}
int launch_fold_wide(const FoldParams &p, unsigned nseg, size_t max_len, int dtype, int op, bool roles,
                     hipStream_t stream, const ChainScratch *chain, size_t displ_bytes) {
  return group(p, nseg, max_len, dtype, op, roles, stream, chain, displ_bytes);
}
}  // namespace alamd
