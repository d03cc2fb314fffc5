// Instantiates residual add + LayerNorm (s = x + r), forward and backward, wide rows.
#include "kernel_table.hpp"

namespace tt {
KernelInfo resnorm_plain_kernel(bool backward, int idx, bool full) { return lookup_res<false>(backward, idx, full); }
}  // namespace tt
