// Instantiates RMSNorm + rotary embedding (forward and backward, wide rows).
#include "kernel_table.hpp"

namespace tt {
KernelInfo rms_rope_kernel(bool backward, int idx, bool full) { return lookup_rope(backward, idx, full); }
}  // namespace tt
