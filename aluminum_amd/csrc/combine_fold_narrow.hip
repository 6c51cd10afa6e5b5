// Fold kernels of the 8- and 16-bit integer types.
#include "combine_fold_impl.h"

namespace alamd {
namespace {
ALAMD_FOLD_GROUP(group, case ALAMD_I8: return dispatch_int_op<int8_t>(op, run);
                 case ALAMD_U8: return dispatch_int_op<uint8_t>(op, run);
                 case ALAMD_I16: return dispatch_int_op<int16_t>(op, run);
                 case ALAMD_U16: return dispatch_int_op<uint16_t>(op, run);)
}
int launch_fold_narrow(const FoldParams &p, unsigned nseg, size_t max_len, int dtype, int op, bool roles,
                       hipStream_t stream, const ChainScratch *chain, size_t displ_bytes) {
  return group(p, nseg, max_len, dtype, op, roles, stream, chain, displ_bytes);
}
}  // namespace alamd
