// Fold kernels of the floating-point types, and the entry of the fold family:
// the integer types are built in combine_fold_narrow.hip and combine_fold_wide.hip.
#include "combine_fold_impl.h"

namespace alamd {
namespace {
ALAMD_FOLD_GROUP(group, case ALAMD_F16: return dispatch_fp_op<f16_t>(op, run);
                 case ALAMD_BF16: return dispatch_fp_op<bf16_t>(op, run);
                 case ALAMD_F32: return dispatch_fp_op<float>(op, run);
                 case ALAMD_F64: return dispatch_fp_op<double>(op, run);)
}
int launch_fold_narrow(const FoldParams &p, unsigned nseg, size_t max_len, int dtype, int op, bool roles,
                       hipStream_t stream, const ChainScratch *chain, size_t displ_bytes);
int launch_fold_wide(const FoldParams &p, unsigned nseg, size_t max_len, int dtype, int op, bool roles,
                     hipStream_t stream, const ChainScratch *chain, size_t displ_bytes);

int launch_fold(const FoldParams &p, unsigned nseg, size_t max_len, int dtype, int op, bool acc_is_in,
                hipStream_t stream, const ChainScratch *chain, size_t displ_bytes) {
  // operand roles only matter where a tie or a NaN can pick a side
  const bool roles = acc_is_in && is_float_dtype(dtype) && (op == ALAMD_MIN || op == ALAMD_MAX);
  switch (dtype) {
  case ALAMD_I8: case ALAMD_U8: case ALAMD_I16: case ALAMD_U16:
    return launch_fold_narrow(p, nseg, max_len, dtype, op, roles, stream, chain, displ_bytes);
  case ALAMD_I32: case ALAMD_U32: case ALAMD_I64: case ALAMD_U64:
    return launch_fold_wide(p, nseg, max_len, dtype, op, roles, stream, chain, displ_bytes);
  default:
    return group(p, nseg, max_len, dtype, op, roles, stream, chain, displ_bytes);
  }
}
}  // namespace alamd
