// Tree kernels of one element type (f16).
#include "combine_tree_impl.h"

namespace alamd {
int launch_tree_f16(const TreeParams &p, int slots, unsigned nseg, size_t max_len, int op, hipStream_t stream,
                    const ChainScratch *scratch, size_t displ_bytes) {
  return launch_tree_of<f16_t>(p, slots, nseg, max_len, op, stream, scratch, displ_bytes);
}
}  // namespace alamd
