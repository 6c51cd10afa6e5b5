// Tree kernels of fp32, and the entry of the tree family: the other float
// types are built in combine_tree_f16.hip, combine_tree_bf16.hip and combine_tree_f64.hip.
#include "combine_tree_impl.h"

namespace alamd {
int launch_tree_f16(const TreeParams &p, int slots, unsigned nseg, size_t max_len, int op, hipStream_t stream,
                    const ChainScratch *scratch, size_t displ_bytes);
int launch_tree_bf16(const TreeParams &p, int slots, unsigned nseg, size_t max_len, int op, hipStream_t stream,
                    const ChainScratch *scratch, size_t displ_bytes);
int launch_tree_f64(const TreeParams &p, int slots, unsigned nseg, size_t max_len, int op, hipStream_t stream,
                    const ChainScratch *scratch, size_t displ_bytes);

int launch_tree(const TreeParams &p, int slots, unsigned nseg, size_t max_len, int dtype, int op,
                hipStream_t stream, const ChainScratch *scratch, size_t displ_bytes) {
  switch (dtype) {
  case ALAMD_F16: return launch_tree_f16(p, slots, nseg, max_len, op, stream, scratch, displ_bytes);
  case ALAMD_BF16: return launch_tree_bf16(p, slots, nseg, max_len, op, stream, scratch, displ_bytes);
  case ALAMD_F32: return launch_tree_of<float>(p, slots, nseg, max_len, op, stream, scratch, displ_bytes);
  case ALAMD_F64: return launch_tree_f64(p, slots, nseg, max_len, op, stream, scratch, displ_bytes);
  default: return set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "tree orders are for the float types (dtype %d)", dtype);
  }
}
}  // namespace alamd
