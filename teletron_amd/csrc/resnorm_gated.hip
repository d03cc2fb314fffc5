// Instantiates gated residual add + LayerNorm (s = x + gate * r), forward and backward, wide rows.
#include "kernel_table.hpp"

namespace tt {
KernelInfo resnorm_gated_kernel(bool backward, int idx, bool full) { return lookup_res<true>(backward, idx, full); }
}  // namespace tt
