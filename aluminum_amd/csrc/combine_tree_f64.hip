// Tree kernels of one element type (f64).
#include "combine_tree_impl.h"

namespace alamd {
int launch_tree_f64(const TreeParams &p, int slots, unsigned nseg, size_t max_len, int op, hipStream_t stream,
                    const ChainScratch *scratch, size_t displ_bytes) {
  return launch_tree_of<double>(p, slots, nseg, max_len, op, stream, scratch, displ_bytes);
}
}  // namespace alamd
