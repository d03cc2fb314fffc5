// Instantiates the adaln bwd kernel family (one translation unit per family so they build in parallel).
#include "kernel_table.hpp"

namespace tt {
KernelInfo adaln_bwd_kernel(bool narrow, int idx, bool full) { return lookup_bwd<kAdaLN>(narrow, idx, full); }
}  // namespace tt
